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

}  // extern "C"
