// Row-wise sparse optimizer steps over (unique ids, gradient rows): one wave per row, 128-bit
// loads and stores, the Adagrad row statistic reduced with a wave butterfly.  The ids of one
// call are distinct (they come from the inspector's dedup), so no two waves touch the same row.
#include "common.hpp"

namespace kge {

template <bool ADAGRAD, int V>
__global__ __launch_bounds__(256) void sparse_step_kernel(float *table, float *state, int d, const int64_t *ids,
                                                          const int32_t *num_unique, const float *rows, float lr,
                                                          float eps)
{
    const int lane = threadIdx.x & (kWave - 1);
    const int64_t u = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (u >= num_unique[0]) return;
    const int64_t id = ids[u];
    const float *g = rows + u * (int64_t)d;
    float *w = table + id * (int64_t)d;
    float scale = lr;
    if constexpr (ADAGRAD) {
        float sq = 0.0f;
        for (int j = lane * V; j < d; j += kWave * V) {
            const Vec<V> gv = Vec<V>::load(g + j);
#pragma unroll
            for (int e = 0; e < V; ++e) sq += gv.v[e] * gv.v[e];
        }
        sq = wave_sum(sq);
        const float s = state[id] + sq / (float)d;
        if (lane == 0) state[id] = s;
        scale = lr / (sqrtf(s) + eps);
    }
    for (int j = lane * V; j < d; j += kWave * V) {
        const Vec<V> gv = Vec<V>::load(g + j);
        Vec<V> wv = Vec<V>::load(w + j);
#pragma unroll
        for (int e = 0; e < V; ++e) wv.v[e] -= scale * gv.v[e];
        wv.store(w + j);
    }
}

template <bool ADAGRAD>
static int launch_step(float *table, float *state, int64_t dim, const int64_t *ids, const int32_t *num_unique,
                       int64_t capacity, const float *rows, float lr, float eps, hipStream_t st)
{
    if (!table || !ids || !num_unique || !rows || (ADAGRAD && !state)) return KGE_EINVAL;
    if (dim <= 0 || dim > (1 << 20) || capacity < 0) return KGE_ESHAPE;
    if (capacity == 0) return KGE_OK;
    const dim3 grid((unsigned)ceil_div(capacity, 4)), block(256);
    if (dim % 4 == 0 && aligned16(table) && aligned16(rows))
        hipLaunchKernelGGL((sparse_step_kernel<ADAGRAD, 4>), grid, block, 0, st, table, state, (int)dim, ids, num_unique,
                           rows, lr, eps);
    else
        hipLaunchKernelGGL((sparse_step_kernel<ADAGRAD, 1>), grid, block, 0, st, table, state, (int)dim, ids, num_unique,
                           rows, lr, eps);
    KGE_CHECK_LAUNCH();
    return KGE_OK;
}

// ---- projection table (TransR / RESCAL) from partly factored gradients -----------------------------
// One workgroup per relation group u.  A dense group streams its d x d gradient row against the
// projection; a factored group (at most four triples, rows x_p / q_p) forms each 128-bit piece of
// sum_p x_p^T q_p in registers while it streams the projection, so the d x d gradient never exists in
// memory.  Adagrad's statistic of a factored group is the Frobenius norm of that sum, from the two
// 4 x 4 Gram matrices of the rows.
__device__ __forceinline__ float block_sum_256(float v, float *s_red)
{
    v = wave_sum(v);
    __syncthreads();  // s_red may still be read from the call before
    if ((threadIdx.x & (kWave - 1)) == 0) s_red[threadIdx.x >> 6] = v;
    __syncthreads();
    return (s_red[0] + s_red[1]) + (s_red[2] + s_red[3]);
}

template <bool ADAGRAD>
__global__ __launch_bounds__(256) void proj_step_kernel(float *proj, float *state, int d, const int64_t *ids,
                                                        const int32_t *num_unique, const int32_t *seg_offsets,
                                                        const float *rows, const float *fx, const float *fq, int fmax,
                                                        float lr, float eps)
{
    extern __shared__ __align__(16) float lds[];  // factored groups: x[0..3][k] as d float4
    __shared__ float s_red[4];
    const int u = blockIdx.x, tid = threadIdx.x;
    if (u >= num_unique[0]) return;
    const int64_t id = ids[u];
    const int s0 = seg_offsets[u], n = seg_offsets[u + 1] - s0;
    const bool factored = fx && n <= fmax;
    const int nq4 = d >> 2;
    const int64_t q4 = (int64_t)d * nq4;  // float4 per matrix
    float4 *M = reinterpret_cast<float4 *>(proj + id * (int64_t)d * d);
    float scale = lr;
    if constexpr (ADAGRAD) {
        float sq = 0.0f;
        if (factored) {
            // ||sum_p x_p^T q_p||_F^2 = sum_{p,p'} (x_p . x_p')(q_p . q_p')
            for (int a = 0; a < n; ++a)
                for (int b = a; b < n; ++b) {
                    float xx = 0.0f, qq = 0.0f;
                    for (int j = tid; j < d; j += 256) {
                        xx = fmaf(fx[(int64_t)(s0 + a) * d + j], fx[(int64_t)(s0 + b) * d + j], xx);
                        qq = fmaf(fq[(int64_t)(s0 + a) * d + j], fq[(int64_t)(s0 + b) * d + j], qq);
                    }
                    xx = block_sum_256(xx, s_red);
                    qq = block_sum_256(qq, s_red);
                    sq += (a == b ? 1.0f : 2.0f) * xx * qq;
                }
        } else {
            const float4 *g = reinterpret_cast<const float4 *>(rows + (int64_t)u * d * d);
            float part = 0.0f;
            for (int64_t f = tid; f < q4; f += 256) {
                const float4 v = g[f];
                part = fmaf(v.x, v.x, fmaf(v.y, v.y, fmaf(v.z, v.z, fmaf(v.w, v.w, part))));
            }
            sq = block_sum_256(part, s_red);
        }
        const float st = state[id] + sq / ((float)d * (float)d);
        __syncthreads();  // every thread has read the old state
        if (tid == 0) state[id] = st;
        scale = lr / (sqrtf(st) + eps);
    }
    if (!factored) {
        const float4 *g = reinterpret_cast<const float4 *>(rows + (int64_t)u * d * d);
        for (int64_t f = tid; f < q4; f += 256) {
            const float4 v = g[f];
            float4 m = M[f];
            m.x -= scale * v.x, m.y -= scale * v.y, m.z -= scale * v.z, m.w -= scale * v.w;
            M[f] = m;
        }
        return;
    }
    float4 *sXT = reinterpret_cast<float4 *>(lds);
    for (int f = tid; f < 4 * nq4; f += 256) {
        const int r = f / nq4, k4 = (f % nq4) * 4;
        const float4 v = r < n ? *reinterpret_cast<const float4 *>(fx + (int64_t)(s0 + r) * d + k4) : make_float4(0.f, 0.f, 0.f, 0.f);
        float *col = reinterpret_cast<float *>(sXT + k4) + r;
        col[0] = v.x, col[4] = v.y, col[8] = v.z, col[12] = v.w;
    }
    const int P = 256 / nq4 > 0 ? 256 / nq4 : 1;
    const int cq = tid % nq4, ph = tid / nq4;
    float4 q[4];
#pragma unroll
    for (int r = 0; r < 4; ++r)
        q[r] = r < n ? *reinterpret_cast<const float4 *>(fq + (int64_t)(s0 + r) * d + 4 * cq) : make_float4(0.f, 0.f, 0.f, 0.f);
    __syncthreads();
    if (ph >= P) return;
    for (int k = ph; k < d; k += P) {
        const float4 x = sXT[k];
        float4 o, m = M[(int64_t)k * nq4 + cq];
        o.x = fmaf(x.w, q[3].x, fmaf(x.z, q[2].x, fmaf(x.y, q[1].x, x.x * q[0].x)));
        o.y = fmaf(x.w, q[3].y, fmaf(x.z, q[2].y, fmaf(x.y, q[1].y, x.x * q[0].y)));
        o.z = fmaf(x.w, q[3].z, fmaf(x.z, q[2].z, fmaf(x.y, q[1].z, x.x * q[0].z)));
        o.w = fmaf(x.w, q[3].w, fmaf(x.z, q[2].w, fmaf(x.y, q[1].w, x.x * q[0].w)));
        m.x -= scale * o.x, m.y -= scale * o.y, m.z -= scale * o.z, m.w -= scale * o.w;
        M[(int64_t)k * nq4 + cq] = m;
    }
}

template <bool ADAGRAD>
static int launch_proj_step(float *proj, float *state, int64_t dim, const kge_inspection *ri, const kge_grads *g, float lr,
                            float eps, hipStream_t st)
{
    if (!proj || !ri || !g || !g->aux_rows || (ADAGRAD && !state)) return KGE_EINVAL;
    if (!ri->unique_ids || !ri->num_unique || !ri->seg_offsets) return KGE_EINVAL;
    if (dim <= 0 || dim % 4 != 0 || dim > (1 << 15) || ri->n < 0) return KGE_ESHAPE;
    if (g->aux_factor_max < 0 || g->aux_factor_max > 4) return KGE_EINVAL;
    const bool factored = g->aux_factor_max > 0;
    if (factored && (!g->aux_x || !g->aux_q)) return KGE_EINVAL;
    if (factored && dim > 1024) return KGE_EUNSUPPORTED;  // (a factored group's column quads are one per thread)
    if (!aligned16(proj) || !aligned16(g->aux_rows) || (factored && (!aligned16(g->aux_x) || !aligned16(g->aux_q)))) return KGE_EINVAL;
    if (ri->n == 0) return KGE_OK;
    const size_t lds = factored ? sizeof(float) * 4 * (size_t)dim : 0;
    hipLaunchKernelGGL((proj_step_kernel<ADAGRAD>), dim3((unsigned)ri->n), dim3(256), lds, st, proj, state, (int)dim,
                       ri->unique_ids, ri->num_unique, ri->seg_offsets, g->aux_rows, factored ? g->aux_x : nullptr,
                       factored ? g->aux_q : nullptr, g->aux_factor_max, lr, eps);
    KGE_CHECK_LAUNCH();
    return KGE_OK;
}

}  // namespace kge

using namespace kge;

extern "C" {

int kge_sparse_sgd(float *table, int64_t dim, const int64_t *ids, const int32_t *num_unique, int64_t capacity,
                   const float *rows, float lr, void *stream)
{
    return launch_step<false>(table, nullptr, dim, ids, num_unique, capacity, rows, lr, 0.0f, as_stream(stream));
}

int kge_sparse_adagrad(float *table, float *state, int64_t dim, const int64_t *ids, const int32_t *num_unique,
                       int64_t capacity, const float *rows, float lr, float eps, void *stream)
{
    return launch_step<true>(table, state, dim, ids, num_unique, capacity, rows, lr, eps, as_stream(stream));
}

int kge_sparse_sgd_factored(float *proj, int64_t dim, const kge_inspection *rel_insp, const kge_grads *grads, float lr,
                            void *stream)
{
    return launch_proj_step<false>(proj, nullptr, dim, rel_insp, grads, lr, 0.0f, as_stream(stream));
}

int kge_sparse_adagrad_factored(float *proj, float *state, int64_t dim, const kge_inspection *rel_insp,
                                const kge_grads *grads, float lr, float eps, void *stream)
{
    return launch_proj_step<true>(proj, state, dim, rel_insp, grads, lr, eps, as_stream(stream));
}

}  // extern "C"
