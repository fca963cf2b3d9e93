// TransR / RESCAL: per-relation projections as grouped dense contractions on fp32 MFMA.
//
// The reference's kernel gives every triple its own vector x matrix product
// (apps/kge/kge.py:321-343, bvm(vh - vt, Proj[r]) + vr; RESCAL kge.py:369-390) and re-reads
// the 4*d*d-byte projection per triple.  Here the triples are grouped by relation (relation
// inspection: sorted order + segment offsets) and every group is multiplied against its
// projection once, 32 triples at a time, with v_mfma_f32_16x16x4_f32.
//
// MFMA operand layout (wave64, 16x16x4 fp32): lane l supplies A[i = l % 16][k = l / 16] and
// B[k = l / 16][j = l % 16]; it receives D[i = 4 * (l / 16) + r][j = l % 16], r = 0..3.
// Two re-labelings keep every memory access 128 bits wide:
//   * k: inside a "superstep" of 16 consecutive k the MFMA step s (0..3) pairs lane group
//     kk = l / 16 with k = 16 q + 4 kk + s, so a lane's A values for the four steps are one
//     float4 of the staged row;
//   * j: a lane's float4 of four consecutive matrix columns feeds four MFMAs (one per element),
//     so MFMA e owns columns n0 + 4 (l % 16) + e.
#include "common.hpp"
#include "seg_reduce.hpp"

namespace kge {

typedef float floatx4 __attribute__((ext_vector_type(4)));

constexpr int kTM = 32;          // triples per tile
#ifndef KGE_TR_RING
#define KGE_TR_RING 2
#endif
#ifndef KGE_TR_OCC
#define KGE_TR_OCC 3
#endif
constexpr int kRing = KGE_TR_RING;  // supersteps of B operands kept in flight per wave
constexpr int kMaxDimMfma = 1024;

int launch_score_pos(const kge_tables *, const kge_batch *, float *, float *, float *, hipStream_t);

// ---- tile plan: one entry per (relation group, block of `tile` sorted positions) -----------
struct TilePlan {
    int32_t *num_tiles;  // [1]
    int32_t *tile_seg;   // [max_tiles] group (unique-relation index)
    int32_t *tile_p0;    // [max_tiles] first sorted position
    // groups longer than one tile ("split" groups, used by the dM kernel): every tile of such
    // a group writes a partial result to slot tile_part[tile]; -1 for unsplit groups
    int32_t *tile_part;   // [max_tiles] or null
    int32_t *num_split;   // [1]
    int32_t *split_seg;   // [max_split] group of the split
    int32_t *split_first; // [max_split] first partial slot
    int32_t *split_cnt;   // [max_split] number of partial slots
};

__device__ int block_inclusive_scan_1024(int v, int *s_scan)
{
    s_scan[threadIdx.x] = v;
    __syncthreads();
    for (int o = 1; o < 1024; o <<= 1) {  // Hillis-Steele
        const int u = (int)threadIdx.x >= o ? s_scan[threadIdx.x - o] : 0;
        __syncthreads();
        s_scan[threadIdx.x] += u;
        __syncthreads();
    }
    const int r = s_scan[threadIdx.x];
    __syncthreads();
    return r;
}

__global__ __launch_bounds__(1024) void transr_plan_kernel(const int32_t *num_unique, const int32_t *seg_offsets,
                                                          TilePlan plan, int tile)
{
    __shared__ int s_scan[1024];
    __shared__ int s_carry[3];
    const int U = num_unique[0];
    if (threadIdx.x < 3) s_carry[threadIdx.x] = 0;
    __syncthreads();
    for (int base = 0; base < U; base += 1024) {
        const int g = base + threadIdx.x;
        int s0 = 0, cnt = 0;
        if (g < U) {
            s0 = seg_offsets[g];
            cnt = (seg_offsets[g + 1] - s0 + tile - 1) / tile;
        }
        const int inc_t = block_inclusive_scan_1024(cnt, s_scan);
        const int start = s_carry[0] + inc_t - cnt;
        int pstart = -1;
        if (plan.tile_part) {
            const int pc = cnt > 1 ? cnt : 0, sg = cnt > 1 ? 1 : 0;
            const int inc_p = block_inclusive_scan_1024(pc, s_scan);
            const int inc_s = block_inclusive_scan_1024(sg, s_scan);
            if (sg) {
                pstart = s_carry[1] + inc_p - pc;
                const int si = s_carry[2] + inc_s - 1;
                plan.split_seg[si] = g;
                plan.split_first[si] = pstart;
                plan.split_cnt[si] = cnt;
            }
            __syncthreads();
            if (threadIdx.x == 1023) s_carry[1] += inc_p, s_carry[2] += inc_s;
        }
        for (int q = 0; q < cnt; ++q) {
            plan.tile_seg[start + q] = g;
            plan.tile_p0[start + q] = s0 + q * tile;
            if (plan.tile_part) plan.tile_part[start + q] = pstart >= 0 ? pstart + q : -1;
        }
        __syncthreads();
        if (threadIdx.x == 1023) s_carry[0] += inc_t;
        __syncthreads();
    }
    if (threadIdx.x == 0) {
        plan.num_tiles[0] = s_carry[0];
        if (plan.num_split) plan.num_split[0] = s_carry[2];
    }
}

// ---- grouped GEMM tile: Y[32 x d] = X[32 x d] * M (or * M^T) -----------------------------
struct GemmArgs {
    const float *ent, *rel, *proj;
    const int64_t *h, *r, *t;
    const int32_t *perm, *seg_offsets;
    const int64_t *unique_ids;
    TilePlan plan;
    const float *xs;  // TRANSPOSED pass: left operand rows in sorted order [B, d]
    float *pos;       // forward: [B] scores (nullable)
    float *resid;     // forward: [B, d] rows y (nullable)
    float *occ_h, *occ_t;  // backward-dX: [B, d] each (occ_t nullable)
    int d, norm_p;
};

// MODE 0: forward TransR   x = E[h]-E[t], y = x M + R[r], score = ||y||_p
// MODE 1: forward RESCAL   x = E[h],      y = x M,        score = y . E[t]
// MODE 2: backward dX      x = xs rows,   y = x M^T -> occ_h = y, occ_t = -y (when occ_t is set)
template <int MODE>
__global__ __launch_bounds__(256, KGE_TR_OCC) void transr_gemm_kernel(GemmArgs a)
{
    extern __shared__ __align__(16) float lds[];
    const int tile = blockIdx.x;
    if (tile >= a.plan.num_tiles[0]) return;
    const int d = a.d;
    const int kpad = (d + 15) & ~15;
    const int pitch = kpad + 4;
    float *sX = lds;                 // [kTM][pitch]
    float *sRed = lds + kTM * pitch; // [4][kTM]
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int g = a.plan.tile_seg[tile], p0 = a.plan.tile_p0[tile];
    const int seg_end = a.seg_offsets[g + 1];
    const int rows = seg_end - p0 < kTM ? seg_end - p0 : kTM;
    const int64_t rid = a.unique_ids[g];
    const float *M = a.proj + rid * (int64_t)d * d;

    // triple ids of the tile first (one dependent-load chain per row instead of one per element)
    __shared__ int s_b[kTM];
    __shared__ int64_t s_h[kTM], s_t[kTM];
    if (tid < kTM) {
        const int b = tid < rows ? a.perm[p0 + tid] : 0;
        s_b[tid] = b;
        if constexpr (MODE != 2) {
            s_h[tid] = a.h[b];
            s_t[tid] = a.t[b];
        }
    }
    __syncthreads();
    // stage the left operand with all loads of a thread in flight together
    {
        const int per_row = kpad / 4;
        constexpr int kStageBatch = 4;
        for (int f0 = tid; f0 < kTM * per_row; f0 += 256 * kStageBatch) {
            float4 v[kStageBatch], u[kStageBatch];
#pragma unroll
            for (int q = 0; q < kStageBatch; ++q) {
                const int f = f0 + 256 * q;
                const int row = f / per_row, k4 = (f % per_row) * 4;
                v[q] = make_float4(0.f, 0.f, 0.f, 0.f), u[q] = v[q];
                if (f < kTM * per_row && row < rows && k4 < d) {
                    if constexpr (MODE == 2) {
                        v[q] = *reinterpret_cast<const float4 *>(a.xs + (int64_t)(p0 + row) * d + k4);
                    } else {
                        v[q] = *reinterpret_cast<const float4 *>(a.ent + s_h[row] * (int64_t)d + k4);
                        if constexpr (MODE == 0)
                            u[q] = *reinterpret_cast<const float4 *>(a.ent + s_t[row] * (int64_t)d + k4);
                    }
                }
            }
#pragma unroll
            for (int q = 0; q < kStageBatch; ++q) {
                const int f = f0 + 256 * q;
                if (f < kTM * per_row) {
                    const int row = f / per_row, k4 = (f % per_row) * 4;
                    *reinterpret_cast<float4 *>(&sX[row * pitch + k4]) =
                        make_float4(v[q].x - u[q].x, v[q].y - u[q].y, v[q].z - u[q].z, v[q].w - u[q].w);
                }
            }
        }
    }
    __syncthreads();

    const int li = lane & 15, kk = lane >> 4;
    const bool two_blocks = rows > 16;
    const bool tiny = rows <= 4;
    float rowsum[8];  // norm / dot partials for rows 4*kk + r (+16)
#pragma unroll
    for (int r = 0; r < 8; ++r) rowsum[r] = 0.0f;

    for (int c0 = 0; c0 < d; c0 += 256) {  // 256 output columns per sweep, split over the waves
        const int span = d - c0 < 256 ? d - c0 : 256;
        const int cw = ((span / 4 + 3) / 4) * 4;  // columns per wave, a multiple of 4
        const int n0 = c0 + wave * cw;
        const int wcols = n0 >= c0 + span ? 0 : (c0 + span - n0 < cw ? c0 + span - n0 : cw);
        floatx4 acc_lo[4], acc_hi[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) acc_lo[e] = floatx4{0.f, 0.f, 0.f, 0.f}, acc_hi[e] = floatx4{0.f, 0.f, 0.f, 0.f};

        if (wcols > 0) {
            const int nq = kpad / 16;
            if constexpr (MODE != 2) {
                // B[k][j] = M[k][n0 + 4 li + e]: one float4 per (k) row per lane
                const bool colok = 4 * li < wcols;
                auto loadb = [&](int q, float4 *dst) {
#pragma unroll
                    for (int s = 0; s < 4; ++s) {
                        const int k = 16 * q + 4 * kk + s;
                        dst[s] = (colok && k < d) ? *reinterpret_cast<const float4 *>(M + (int64_t)k * d + n0 + 4 * li)
                                                  : make_float4(0.f, 0.f, 0.f, 0.f);
                    }
                };
                float4 ring[kRing][4];  // supersteps of B in flight
#pragma unroll
                for (int u = 0; u < kRing; ++u)
                    if (u < nq) loadb(u, ring[u]);
                for (int q = 0; q < nq; q += kRing) {
#pragma unroll
                    for (int u = 0; u < kRing; ++u) {
                        if (q + u >= nq) break;
                        float4 bc[4];
#pragma unroll
                        for (int s = 0; s < 4; ++s) bc[s] = ring[u][s];
                        if (q + u + kRing < nq) loadb(q + u + kRing, ring[u]);
                        const int qq = q + u;
                        if (tiny) {
                            // <= 4 triples: plain FMAs beat a 16-row MFMA block that is 3/4 padding.
                            // Lane group kk covers its four k of the superstep; the groups are summed
                            // after the loop.  acc_lo[e][r] = row r, column n0 + 4 li + e.
#pragma unroll
                            for (int r = 0; r < 4; ++r) {
                                if (r >= rows) break;
                                const float4 xr = *reinterpret_cast<const float4 *>(&sX[r * pitch + 16 * qq + 4 * kk]);
                                const float xs4[4] = {xr.x, xr.y, xr.z, xr.w};
#pragma unroll
                                for (int s = 0; s < 4; ++s) {
                                    acc_lo[0][r] = fmaf(xs4[s], bc[s].x, acc_lo[0][r]);
                                    acc_lo[1][r] = fmaf(xs4[s], bc[s].y, acc_lo[1][r]);
                                    acc_lo[2][r] = fmaf(xs4[s], bc[s].z, acc_lo[2][r]);
                                    acc_lo[3][r] = fmaf(xs4[s], bc[s].w, acc_lo[3][r]);
                                }
                            }
                            continue;
                        }
                        const float4 alo = *reinterpret_cast<const float4 *>(&sX[li * pitch + 16 * qq + 4 * kk]);
                        const float4 ahi = *reinterpret_cast<const float4 *>(&sX[(16 + li) * pitch + 16 * qq + 4 * kk]);
                        const float al[4] = {alo.x, alo.y, alo.z, alo.w}, ah[4] = {ahi.x, ahi.y, ahi.z, ahi.w};
#pragma unroll
                        for (int s = 0; s < 4; ++s) {
                            const float bv[4] = {bc[s].x, bc[s].y, bc[s].z, bc[s].w};
#pragma unroll
                            for (int e = 0; e < 4; ++e) {
                                acc_lo[e] = __builtin_amdgcn_mfma_f32_16x16x4f32(al[s], bv[e], acc_lo[e], 0, 0, 0);
                                if (two_blocks)
                                    acc_hi[e] = __builtin_amdgcn_mfma_f32_16x16x4f32(ah[s], bv[e], acc_hi[e], 0, 0, 0);
                            }
                        }
                    }
                }
            } else {
                // B[k][j] = M[j][k] (transposed): MFMA e owns output columns n0 + 16 e + li, and a
                // lane's float4 along k of row (n0 + 16 e + li) serves the four steps
                auto loadb = [&](int q, float4 *dst) {
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        const int col = 16 * e + li, k = 16 * q + 4 * kk;
                        dst[e] = (col < wcols && k < d)
                                     ? *reinterpret_cast<const float4 *>(M + (int64_t)(n0 + col) * d + k)
                                     : make_float4(0.f, 0.f, 0.f, 0.f);
                    }
                };
                float4 ring[kRing][4];
#pragma unroll
                for (int u = 0; u < kRing; ++u)
                    if (u < nq) loadb(u, ring[u]);
                for (int q = 0; q < nq; q += kRing) {
#pragma unroll
                    for (int u = 0; u < kRing; ++u) {
                        if (q + u >= nq) break;
                        float4 bc[4];
#pragma unroll
                        for (int e = 0; e < 4; ++e) bc[e] = ring[u][e];
                        if (q + u + kRing < nq) loadb(q + u + kRing, ring[u]);
                        const int qq = q + u;
                        if (tiny) {  // acc_lo[e][r] = row r, column n0 + 16 e + li
#pragma unroll
                            for (int r = 0; r < 4; ++r) {
                                if (r >= rows) break;
                                const float4 xr = *reinterpret_cast<const float4 *>(&sX[r * pitch + 16 * qq + 4 * kk]);
#pragma unroll
                                for (int e = 0; e < 4; ++e)
                                    acc_lo[e][r] = fmaf(xr.x, bc[e].x, fmaf(xr.y, bc[e].y,
                                                   fmaf(xr.z, bc[e].z, fmaf(xr.w, bc[e].w, acc_lo[e][r]))));
                            }
                            continue;
                        }
                        const float4 alo = *reinterpret_cast<const float4 *>(&sX[li * pitch + 16 * qq + 4 * kk]);
                        const float4 ahi = *reinterpret_cast<const float4 *>(&sX[(16 + li) * pitch + 16 * qq + 4 * kk]);
                        const float al[4] = {alo.x, alo.y, alo.z, alo.w}, ah[4] = {ahi.x, ahi.y, ahi.z, ahi.w};
#pragma unroll
                        for (int e = 0; e < 4; ++e) {
                            const float bv[4] = {bc[e].x, bc[e].y, bc[e].z, bc[e].w};
#pragma unroll
                            for (int s = 0; s < 4; ++s) {
                                acc_lo[e] = __builtin_amdgcn_mfma_f32_16x16x4f32(al[s], bv[s], acc_lo[e], 0, 0, 0);
                                if (two_blocks)
                                    acc_hi[e] = __builtin_amdgcn_mfma_f32_16x16x4f32(ah[s], bv[s], acc_hi[e], 0, 0, 0);
                            }
                        }
                    }
                }
            }
        }

        if (tiny) {  // sum the four k-slices; every lane group then holds rows 0..3 (group 0 writes)
#pragma unroll
            for (int e = 0; e < 4; ++e)
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    float v = acc_lo[e][r];
                    v += __shfl_xor(v, 16, kWave);
                    v += __shfl_xor(v, 32, kWave);
                    acc_lo[e][r] = v;
                }
        }
        // epilogue for this sweep: lane holds rows 4 kk + r (and +16), columns per the mode
#pragma unroll
        for (int blk = 0; blk < 2; ++blk) {
            if (blk == 1 && !two_blocks) break;
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int row = 16 * blk + 4 * kk + r;
                if (row >= rows) continue;
                const int b = s_b[row];
                float y[4];
#pragma unroll
                for (int e = 0; e < 4; ++e) y[e] = blk ? acc_hi[e][r] : acc_lo[e][r];
                if constexpr (MODE != 2) {
                    const int col = n0 + 4 * li;  // y[e] is column col + e
                    if (4 * li < wcols) {
                        if constexpr (MODE == 0) {
                            const float4 rv = *reinterpret_cast<const float4 *>(a.rel + rid * (int64_t)d + col);
                            y[0] += rv.x, y[1] += rv.y, y[2] += rv.z, y[3] += rv.w;
                            float s = 0.0f;
#pragma unroll
                            for (int e = 0; e < 4; ++e) s += a.norm_p == 1 ? fabsf(y[e]) : y[e] * y[e];
                            rowsum[4 * blk + r] += s;
                        } else {
                            const float4 tv = *reinterpret_cast<const float4 *>(a.ent + s_t[row] * (int64_t)d + col);
                            rowsum[4 * blk + r] += y[0] * tv.x + y[1] * tv.y + y[2] * tv.z + y[3] * tv.w;
                        }
                        if (a.resid)
                            *reinterpret_cast<float4 *>(a.resid + (int64_t)b * d + col) =
                                make_float4(y[0], y[1], y[2], y[3]);
                    }
                } else {
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        const int cl = 16 * e + li;
                        if (cl < wcols) {
                            a.occ_h[(int64_t)b * d + n0 + cl] = y[e];
                            if (a.occ_t) a.occ_t[(int64_t)b * d + n0 + cl] = -y[e];
                        }
                    }
                }
            }
        }
    }

    if constexpr (MODE != 2) {
        if (a.pos) {
            // row sums: over the 16 lanes that share kk, then over the four waves
#pragma unroll
            for (int r = 0; r < 8; ++r) {
                float v = rowsum[r];
                v += __shfl_xor(v, 1, kWave);
                v += __shfl_xor(v, 2, kWave);
                v += __shfl_xor(v, 4, kWave);
                v += __shfl_xor(v, 8, kWave);
                if (li == 0) sRed[wave * kTM + 16 * (r >> 2) + 4 * kk + (r & 3)] = v;
            }
            __syncthreads();
            if (tid < rows) {
                const float s = sRed[tid] + sRed[kTM + tid] + sRed[2 * kTM + tid] + sRed[3 * kTM + tid];
                a.pos[s_b[tid]] = (MODE == 0 && a.norm_p == 2) ? sqrtf(s) : s;
            }
        }
    }
}

static size_t gemm_lds_bytes(int d)
{
    const int kpad = (d + 15) & ~15;
    return sizeof(float) * ((size_t)kTM * (kpad + 4) + 4 * kTM);
}

static int64_t max_tiles(const kge_tables *tab, const kge_batch *bat)
{
    const int64_t groups = bat->batch < tab->n_rel ? bat->batch : tab->n_rel;
    return groups + bat->batch / kTM + 1;
}

static bool mfma_path_ok(const kge_tables *tab, const kge_batch *bat)
{
    return bat->rel_insp && tab->dim % 4 == 0 && tab->dim <= kMaxDimMfma && aligned16(tab->ent) &&
           aligned16(tab->aux) && (!tab->rel || aligned16(tab->rel)) && bat->rel_insp->n == bat->batch;
}

// ---- backward kernels ----------------------------------------------------------------------
struct PrepArgs {
    const float *ent;
    const int64_t *h, *t;
    const int32_t *perm;
    const float *dpos, *spos, *resid;
    float *xs, *qs;  // [B, d] in sorted order
    float *occ_t;    // RESCAL: g * v
    int64_t B;
    int d, norm_p, rescal;
};

// One wave per sorted position p (triple b = perm[p]):
//   TransR: xs[p] = E[h]-E[t], qs[p] = g * d||e||/de     RESCAL: xs[p] = E[h], qs[p] = g * E[t], occ_t[b] = g * v
__global__ __launch_bounds__(256) void transr_prep_kernel(PrepArgs a)
{
    const int lane = threadIdx.x & 63;
    const int64_t p = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (p >= a.B) return;
    const int b = a.perm[p];
    const int d = a.d;
    const float g = a.dpos ? a.dpos[b] : 0.0f;
    const float *eh = a.ent + a.h[b] * (int64_t)d, *et = a.ent + a.t[b] * (int64_t)d;
    const float *e = a.resid + (int64_t)b * d;
    float gs = g;
    if (!a.rescal && a.norm_p == 2) {
        const float s = a.spos[b];
        gs = s > 0.0f ? g / s : 0.0f;
    }
    for (int j = lane * 4; j < d; j += 256) {
        const float4 vh = *reinterpret_cast<const float4 *>(eh + j), vt = *reinterpret_cast<const float4 *>(et + j);
        const float4 ve = *reinterpret_cast<const float4 *>(e + j);
        float4 x, q;
        if (a.rescal) {
            x = vh;
            q = make_float4(g * vt.x, g * vt.y, g * vt.z, g * vt.w);
            *reinterpret_cast<float4 *>(a.occ_t + (int64_t)b * d + j) = make_float4(g * ve.x, g * ve.y, g * ve.z, g * ve.w);
        } else {
            x = make_float4(vh.x - vt.x, vh.y - vt.y, vh.z - vt.z, vh.w - vt.w);
            if (a.norm_p == 1) q = make_float4(gs * sgn(ve.x), gs * sgn(ve.y), gs * sgn(ve.z), gs * sgn(ve.w));
            else q = make_float4(gs * ve.x, gs * ve.y, gs * ve.z, gs * ve.w);
        }
        *reinterpret_cast<float4 *>(a.xs + p * d + j) = x;
        *reinterpret_cast<float4 *>(a.qs + p * d + j) = q;
    }
}

constexpr int kDmChunk = 256;  // triples of one relation group per dM work item

struct DmArgs {
    const float *xs, *qs;  // sorted order [B, d]
    const int32_t *seg_offsets;
    TilePlan plan;   // tiles of kDmChunk positions, with split bookkeeping
    float *dm;       // [U, d, d]
    float *part;     // [max_slots, d, d] partial results of split groups
    int d;
};

// dM[g][i][j] = sum_{p in group g} xs[p][i] * qs[p][j].  A work item is (chunk of <= 256 triples
// of one group, 32 rows i); the four waves split the columns j; K runs over the chunk's triples,
// operands prefetched four supersteps ahead.  Groups longer than one chunk write per-chunk
// partial matrices that transr_dm_finish_kernel adds up (keeps the longest K loop at 16 supersteps).
__global__ __launch_bounds__(256, KGE_TR_OCC) void transr_dm_kernel(DmArgs a)
{
    const int d = a.d;
    const int nib = (d + 31) / 32;
    const int tile = blockIdx.x / nib;
    if (tile >= a.plan.num_tiles[0]) return;
    const int i0 = (blockIdx.x % nib) * 32;
    const int g = a.plan.tile_seg[tile];
    const int s0 = a.plan.tile_p0[tile];
    const int seg_end = a.seg_offsets[g + 1];
    const int s1 = s0 + kDmChunk < seg_end ? s0 + kDmChunk : seg_end;
    const int slot = a.plan.tile_part[tile];
    float *dst = slot >= 0 ? a.part + (int64_t)slot * d * d : a.dm + (int64_t)g * d * d;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int li = lane & 15, kk = lane >> 4;
    const bool two_blocks = i0 + 16 < d;
    const bool ilo = i0 + li < d, ihi = i0 + 16 + li < d;
    const int nq = (s1 - s0 + 15) / 16;

    for (int c0 = 0; c0 < d; c0 += 256) {
        const int span = d - c0 < 256 ? d - c0 : 256;
        const int cw = ((span / 4 + 3) / 4) * 4;
        const int n0 = c0 + wave * cw;
        const int wcols = n0 >= c0 + span ? 0 : (c0 + span - n0 < cw ? c0 + span - n0 : cw);
        if (wcols <= 0) continue;
        const bool colok = 4 * li < wcols;
        floatx4 acc_lo[4], acc_hi[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) acc_lo[e] = floatx4{0.f, 0.f, 0.f, 0.f}, acc_hi[e] = floatx4{0.f, 0.f, 0.f, 0.f};

        struct Stage {
            float al[4], ah[4];
            float4 bv[4];
        };
        auto load_stage = [&](int q, Stage &st) {
#pragma unroll
            for (int s = 0; s < 4; ++s) {
                const int p = s0 + 16 * q + 4 * kk + s;
                const bool ok = p < s1;
                const float *xr = a.xs + (int64_t)p * d + i0;
                st.al[s] = (ok && ilo) ? xr[li] : 0.0f;
                st.ah[s] = (ok && ihi) ? xr[16 + li] : 0.0f;
                st.bv[s] = (ok && colok) ? *reinterpret_cast<const float4 *>(a.qs + (int64_t)p * d + n0 + 4 * li)
                                         : make_float4(0.f, 0.f, 0.f, 0.f);
            }
        };
        Stage ring[kRing];
#pragma unroll
        for (int u = 0; u < kRing; ++u)
            if (u < nq) load_stage(u, ring[u]);
        for (int q = 0; q < nq; q += kRing) {
#pragma unroll
            for (int u = 0; u < kRing; ++u) {
                if (q + u >= nq) break;
                const Stage cur = ring[u];
                if (q + u + kRing < nq) load_stage(q + u + kRing, ring[u]);
#pragma unroll
                for (int s = 0; s < 4; ++s) {
                    const float b4[4] = {cur.bv[s].x, cur.bv[s].y, cur.bv[s].z, cur.bv[s].w};
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        acc_lo[e] = __builtin_amdgcn_mfma_f32_16x16x4f32(cur.al[s], b4[e], acc_lo[e], 0, 0, 0);
                        if (two_blocks)
                            acc_hi[e] = __builtin_amdgcn_mfma_f32_16x16x4f32(cur.ah[s], b4[e], acc_hi[e], 0, 0, 0);
                    }
                }
            }
        }
        if (colok) {
#pragma unroll
            for (int blk = 0; blk < 2; ++blk)
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const int row = i0 + 16 * blk + 4 * kk + r;
                    if (row >= d) continue;
                    float4 v;
                    if (blk == 0) v = make_float4(acc_lo[0][r], acc_lo[1][r], acc_lo[2][r], acc_lo[3][r]);
                    else v = make_float4(acc_hi[0][r], acc_hi[1][r], acc_hi[2][r], acc_hi[3][r]);
                    *reinterpret_cast<float4 *>(dst + (int64_t)row * d + n0 + 4 * li) = v;
                }
        }
    }
}

// dM of a split group = sum of its partial matrices (slot order = ascending chunk order)
__global__ __launch_bounds__(256) void transr_dm_finish_kernel(DmArgs a)
{
    const int sidx = blockIdx.y;
    if (sidx >= a.plan.num_split[0]) return;
    const int64_t dd4 = (int64_t)a.d * a.d / 4;
    const int64_t f = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (f >= dd4) return;
    const int g = a.plan.split_seg[sidx], first = a.plan.split_first[sidx], cnt = a.plan.split_cnt[sidx];
    const float4 *src = reinterpret_cast<const float4 *>(a.part) + (int64_t)first * dd4 + f;
    float4 acc = src[0];
    for (int c = 1; c < cnt; ++c) {
        const float4 v = src[(int64_t)c * dd4];
        acc.x += v.x, acc.y += v.y, acc.z += v.z, acc.w += v.w;
    }
    reinterpret_cast<float4 *>(a.dm)[(int64_t)g * dd4 + f] = acc;
}

// ---- host side -----------------------------------------------------------------------------
static size_t up256(size_t x) { return (x + 255) & ~size_t(255); }

struct RPlan {
    size_t off_plan, off_dplan, off_xs, off_qs, off_occ, off_part_e, off_part_r, off_dpart, total;
    int64_t tiles, dtiles, dsplit, dslots;
};

static size_t plan_ints(int64_t tiles, int64_t split) { return (size_t)(64 + 3 * tiles + 3 * split + 8); }

static RPlan make_rplan(const kge_tables *tab, const kge_batch *bat)
{
    RPlan p{};
    const int64_t B = bat->batch, d = tab->dim;
    const int64_t groups = B < tab->n_rel ? B : tab->n_rel;
    p.tiles = max_tiles(tab, bat);
    p.dtiles = groups + B / kDmChunk + 1;
    p.dsplit = B / kDmChunk + 1;            // a split group has more than kDmChunk triples
    p.dslots = 2 * (B / kDmChunk) + 2;      // sum over split groups of ceil(n_g / chunk)
    size_t o = 0;
    p.off_plan = o, o += up256(sizeof(int32_t) * plan_ints(p.tiles, 0));
    p.off_dplan = o, o += up256(sizeof(int32_t) * plan_ints(p.dtiles, p.dsplit));
    p.off_xs = o, o += up256(sizeof(float) * (size_t)(B * d));
    p.off_qs = o, o += up256(sizeof(float) * (size_t)(B * d));
    p.off_occ = o, o += up256(sizeof(float) * (size_t)(2 * B * d));
    p.off_part_e = o, o += up256(sizeof(float) * (size_t)seg_partial_floats(2 * B, d));
    p.off_part_r = o, o += up256(sizeof(float) * (size_t)seg_partial_floats(B, d));
    p.off_dpart = o, o += up256(sizeof(float) * (size_t)(p.dslots * d * d));
    p.total = o;
    return p;
}

static TilePlan plan_at(void *base, int64_t tiles, int64_t split)
{
    int32_t *q = static_cast<int32_t *>(base);
    TilePlan p{q, q + 64, q + 64 + tiles, nullptr, nullptr, nullptr, nullptr, nullptr};
    if (split > 0) {
        p.tile_part = q + 64 + 2 * tiles;
        p.num_split = q + 32;
        p.split_seg = q + 64 + 3 * tiles;
        p.split_first = p.split_seg + split;
        p.split_cnt = p.split_first + split;
    }
    return p;
}

size_t transr_fwd_workspace(const kge_tables *tab, const kge_batch *bat)
{
    return up256(sizeof(int32_t) * plan_ints(max_tiles(tab, bat), 0));
}

int launch_transr_fwd(const kge_tables *tab, const kge_batch *bat, float *pos, float *resid, void *workspace,
                      size_t workspace_bytes, hipStream_t st)
{
    if (bat->batch == 0) return KGE_OK;
    const bool rescal = tab->model == KGE_RESCAL;
    if (!mfma_path_ok(tab, bat) || !workspace || workspace_bytes < transr_fwd_workspace(tab, bat) ||
        gemm_lds_bytes((int)tab->dim) > 64 * 1024)
        return launch_score_pos(tab, bat, pos, resid, nullptr, st);
    const kge_inspection *ri = bat->rel_insp;
    const int64_t tiles = max_tiles(tab, bat);
    TilePlan plan = plan_at(workspace, tiles, 0);
    hipLaunchKernelGGL(transr_plan_kernel, dim3(1), dim3(1024), 0, st, ri->num_unique, ri->seg_offsets, plan, kTM);
    GemmArgs a{tab->ent, tab->rel, tab->aux, bat->h, bat->r, bat->t, ri->perm, ri->seg_offsets, ri->unique_ids,
               plan, nullptr, pos, resid, nullptr, nullptr, (int)tab->dim, tab->norm_p};
    const size_t lds = gemm_lds_bytes((int)tab->dim);
    if (rescal)
        hipLaunchKernelGGL(transr_gemm_kernel<1>, dim3((unsigned)tiles), dim3(256), lds, st, a);
    else
        hipLaunchKernelGGL(transr_gemm_kernel<0>, dim3((unsigned)tiles), dim3(256), lds, st, a);
    KGE_CHECK_LAUNCH();
    return KGE_OK;
}

size_t transr_bwd_workspace(const kge_tables *tab, const kge_batch *bat) { return make_rplan(tab, bat).total; }

int launch_transr_bwd(const kge_tables *tab, const kge_batch *bat, const kge_saved *saved, const float *dpos,
                      const kge_grads *grads, void *workspace, size_t workspace_bytes, hipStream_t st)
{
    const bool rescal = tab->model == KGE_RESCAL;
    if (bat->neg) return KGE_EUNSUPPORTED;  // positives only for the projection models
    if (!mfma_path_ok(tab, bat) || gemm_lds_bytes((int)tab->dim) > 64 * 1024) return KGE_EUNSUPPORTED;
    if (!saved->residual || !grads->aux_rows || !grads->ent_rows) return KGE_EINVAL;
    if (!rescal && (!grads->rel_rows || (tab->norm_p == 2 && !saved->pos))) return KGE_EINVAL;
    const RPlan p = make_rplan(tab, bat);
    if (!workspace || workspace_bytes < p.total) return KGE_EWORKSPACE;
    if (bat->ent_insp->n != 2 * bat->batch) return KGE_ESHAPE;
    const int64_t B = bat->batch;
    const int d = (int)tab->dim;
    char *ws = static_cast<char *>(workspace);
    float *xs = reinterpret_cast<float *>(ws + p.off_xs), *qs = reinterpret_cast<float *>(ws + p.off_qs);
    float *occ = reinterpret_cast<float *>(ws + p.off_occ);
    const kge_inspection *ri = bat->rel_insp;
    TilePlan plan = plan_at(ws + p.off_plan, p.tiles, 0);
    TilePlan dplan = plan_at(ws + p.off_dplan, p.dtiles, p.dsplit);

    PrepArgs pa{tab->ent, bat->h, bat->t, ri->perm, dpos, saved->pos, saved->residual, xs, qs, occ + B * d, B, d,
                tab->norm_p, rescal ? 1 : 0};
    hipLaunchKernelGGL(transr_prep_kernel, dim3((unsigned)ceil_div(B, 4)), dim3(256), 0, st, pa);
    hipLaunchKernelGGL(transr_plan_kernel, dim3(1), dim3(1024), 0, st, ri->num_unique, ri->seg_offsets, plan, kTM);
    hipLaunchKernelGGL(transr_plan_kernel, dim3(1), dim3(1024), 0, st, ri->num_unique, ri->seg_offsets, dplan,
                       kDmChunk);
    // dX = Q M^T -> occurrence rows of h (and -dX for t)
    GemmArgs ga{tab->ent, tab->rel, tab->aux, bat->h, bat->r, bat->t, ri->perm, ri->seg_offsets, ri->unique_ids,
                plan, qs, nullptr, nullptr, occ, rescal ? nullptr : occ + B * d, d, tab->norm_p};
    hipLaunchKernelGGL(transr_gemm_kernel<2>, dim3((unsigned)p.tiles), dim3(256), gemm_lds_bytes(d), st, ga);
    // dM = X^T Q per relation group
    DmArgs da{xs, qs, ri->seg_offsets, dplan, grads->aux_rows, reinterpret_cast<float *>(ws + p.off_dpart), d};
    hipLaunchKernelGGL(transr_dm_kernel, dim3((unsigned)(ceil_div(d, 32) * p.dtiles)), dim3(256), 0, st, da);
    hipLaunchKernelGGL(transr_dm_finish_kernel, dim3((unsigned)ceil_div((int64_t)d * d / 4, 256), (unsigned)p.dsplit),
                       dim3(256), 0, st, da);
    KGE_CHECK_LAUNCH();
    if (bat->insp_ready && hipStreamWaitEvent(st, reinterpret_cast<hipEvent_t>(bat->insp_ready), 0) != hipSuccess)
        return KGE_ELAUNCH;
    // entity rows from the h / t occurrence rows; dR[g] = sum of the group's q rows, which are
    // already stored in sorted order
    const SegJob jobs[2] = {
        {occ, bat->ent_insp, d, grads->ent_rows, reinterpret_cast<float *>(ws + p.off_part_e), false},
        {qs, ri, d, grads->rel_rows, reinterpret_cast<float *>(ws + p.off_part_r), true}};
    return launch_seg_reduce_jobs(jobs, rescal ? 1 : 2, st);
}

}  // namespace kge
