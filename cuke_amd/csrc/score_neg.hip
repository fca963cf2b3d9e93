// Shared-negative forward: every positive of a chunk against the chunk's N
// negative tails (layout of apps/examples/examples.py:1404-1444, which the
// reference only ever lowers to serial CPU loops).
//
// One workgroup owns a (TB positives x TN negatives) tile of one chunk.  The
// "query" rows a_b = f(h_b, r_b) are formed while staging (the gathers of h and r
// are fused into the staging loads) and the negative rows are gathered straight
// into LDS, KD floats of the row at a time; each thread then accumulates an
// RB x RK block of pair scores from LDS with 128-bit reads (score_neg_kernel, fp32 vector
// ALUs).  Where the pair scores are plain dot products (DistMult, ComplEx, and the w . t'
// sweep of TransH) the tile is a matrix product and runs on the matrix cores
// (score_neg_mfma_kernel, fp32 MFMA with fp32 accumulation).
#include <type_traits>

#include "inspector_mid.hpp"
#include "score_pos_body.hpp"
#include "tile_common.hpp"

namespace kge {

struct NegArgs {
    const float *ent, *rel, *aux;
    const int64_t *h, *r, *neg;  // h: the side of the positive that is kept (tails with head negatives)
    const float *side_pos;  // TransH: w_b . h_b; TransF: r_b . h_b (the kept side: t_b with head negatives)
    const float *query;     // RotatE: rotated heads [B, d] from the positive kernel; RESCAL: projected rows E[h] Proj[r] (required)
    float *out;             // [B, N]
    float *side_neg;        // TransH save-for-backward [2, B, N] (optional):
                            //   plane 0: c = w_b . t'_k ; plane 1: sum_i phi(u_i) w_i with
                            //   phi = sign (L1) or u / ||u|| (L2)
    int64_t plane;          // B * N
    int C, N, d, rel_dim;
    float gamma;
    int vec, n_chunks;
    float rsign;            // +1: negatives replace the tail; -1: the head (see load_query)
    // Small batches: the reduction axis is split over `ksplit` workgroups per tile, each writes the raw
    // sums of its slices to plane `split` of `partial` ([ksplit][B * N]) and score_neg_finish_kernel
    // adds the planes and finishes the scores.  ksplit <= 1: one workgroup per tile, scores written directly.
    int ksplit;
    float *partial;
    // TransE, DistMult / ComplEx on the matrix-core tiles, nothing riding along: the workgroups behind
    // the `tile_blocks` tile workgroups score the positives (their score does not enter the tiles, so
    // the two need not be two launches).  pos_blocks == 0: none.
    PosArgs pos;
    int tile_blocks, pos_blocks;
};

typedef float v4f __attribute__((ext_vector_type(4)));

constexpr int kKD = 32;        // floats of each row staged per step
constexpr int kLDW = kKD + 4;  // LDS row pitch: +4 floats keeps 128-bit reads of
                               // 8 consecutive rows on distinct banks

// One element of the pair update, per model.
template <int MODEL, int P, bool SAVE>
__device__ __forceinline__ void pair_elem(float &acc, float &acc2, float a0, float a1, float t0, float t1,
                                          float c)
{
    if constexpr (MODEL == KGE_DISTMULT || MODEL == KGE_COMPLEX || MODEL == KGE_TRANSF || MODEL == KGE_RESCAL) {
        acc = fmaf(a0, t0, acc);
    } else if constexpr (MODEL == KGE_TRANSE) {
        const float u = a0 - t0;
        if constexpr (P == 1) acc += fabsf(u);
        else acc = fmaf(u, u, acc);
    } else if constexpr (MODEL == KGE_TRANSH) {
        // a0 = h + r - (w.h) w, a1 = w, c = w . t'
        // (P == 1 with SAVE: a0, a1 and t0 carry the factor 2^100, see sgn_of_scaled)
        const float u = fmaf(c, a1, a0 - t0);
        if constexpr (P == 1) acc += fabsf(u);
        else acc = fmaf(u, u, acc);
        if constexpr (SAVE) acc2 = fmaf(P == 1 ? sgn_of_scaled(u) : u, a1, acc2);
    } else if constexpr (MODEL == KGE_ROTATE) {
        const float ur = a0 - t0, ui = a1 - t1;
        acc += __builtin_amdgcn_sqrtf(fmaf(ur, ur, ui * ui));
    }
}

template <int MODEL, int P, int RB, int RK, bool SAVE, bool VEC4>
__global__ __launch_bounds__(256, KGE_TILE_OCC) void score_neg_kernel(NegArgs a, FusedInsp fi)
{
    extern __shared__ __align__(16) char dyn_smem[];
    if (fused_insp_block(fi, reinterpret_cast<uint32_t *>(dyn_smem))) return;
    if constexpr (MODEL == KGE_TRANSE) {  // the positives carried along (NegArgs::pos)
        if (a.pos_blocks > 0 && (int)blockIdx.x - fi.blocks >= a.tile_blocks) {
            score_pos_body<MODEL, P, 4>(a.pos, nullptr, (int64_t)((int)blockIdx.x - fi.blocks - a.tile_blocks));
            return;
        }
    }
    constexpr int TB = 16 * RB, TN = 16 * RK;
    constexpr int NPA = (MODEL == KGE_ROTATE || MODEL == KGE_TRANSH) ? 2 : 1;
    constexpr int NPT = MODEL == KGE_ROTATE ? 2 : 1;
    constexpr int SB = TB / 32, SN = TN / 32;  // float4 per thread per plane per step
    // TransH, L1, with the sign sums saved for backward: the second sweep's rows are staged times
    // 2^100 so that the sign of a residual element is a single clamp (tile_common.hpp)
    constexpr bool kScaled = MODEL == KGE_TRANSH && P == 1 && SAVE;
    static_assert(TB % 32 == 0 && TN % 32 == 0, "tile rows are staged 32 at a time");

    float(*sA)[TB][kLDW] = reinterpret_cast<float(*)[TB][kLDW]>(dyn_smem);
    float(*sT)[TN][kLDW] = reinterpret_cast<float(*)[TN][kLDW]>(dyn_smem + sizeof(float) * NPA * TB * kLDW);

    const int tid = threadIdx.x, tx = tid & 15, ty = tid >> 4;
    const int srow = tid >> 3, scol = (tid & 7) * 4;
    int c, tile_y, tile_x;
    int lid = blockIdx.x - fi.blocks, split = 0;
    if (a.ksplit > 1) {  // (never TransH: its w . t' sweep needs the whole row)
        const int tiles = a.tile_blocks / a.ksplit;  // a multiple of 8: the tile keeps its XCD
        split = lid / tiles, lid -= split * tiles;
    }
    if (!xcd_tile(lid, (a.N + TN - 1) / TN, (a.C + TB - 1) / TB, a.n_chunks, c, tile_y, tile_x)) return;
    const int bt0 = tile_y * TB, kt0 = tile_x * TN;
    const int d = a.d, half = d >> 1;
    const int klen = MODEL == KGE_ROTATE ? half : d;
    // (VEC4, 128-bit row loads, is a compile-time choice: as a run-time one the compiler merges the two
    // forms of the raw loads into the scalar one)

    // rows this thread stages
    const float *ph[SB], *pr[SB], *pw[SB], *pq[SB];
    float pa[SB];
    bool okb[SB];
#pragma unroll
    for (int s = 0; s < SB; ++s) {
        const int bl = bt0 + srow + 32 * s;
        okb[s] = bl < a.C;
        const int64_t b = (int64_t)c * a.C + (okb[s] ? bl : a.C - 1);
        const int64_t rid = a.r[b];
        ph[s] = a.ent + a.h[b] * (int64_t)d;
        pr[s] = a.rel + rid * (int64_t)a.rel_dim;
        pw[s] = MODEL == KGE_TRANSH ? a.aux + rid * (int64_t)d : nullptr;
        pa[s] = MODEL == KGE_TRANSH ? a.side_pos[b] : 0.0f;
        pq[s] = (MODEL == KGE_ROTATE || MODEL == KGE_RESCAL) ? a.query + b * (int64_t)d : nullptr;
    }
    const float *pt[SN];
    bool okk[SN];
#pragma unroll
    for (int s = 0; s < SN; ++s) {
        const int kl = kt0 + srow + 32 * s;
        okk[s] = kl < a.N;
        pt[s] = a.ent + a.neg[(int64_t)c * a.N + (okk[s] ? kl : a.N - 1)] * (int64_t)d;
    }

    // The rows of the next slice are requested as raw operands -- clamped addresses, no select, no
    // arithmetic on what was loaded -- and only become query rows (h o r, h + r - (w.h) w ..., zeros
    // outside the tile) when the slice is written to LDS: anything that touches a loaded register makes
    // the compiler wait for the loads where they are issued, i.e. in front of the compute they are meant
    // to overlap.
    constexpr int NRAW = query_raw_count<MODEL>();
    float4 qraw[SB][NRAW], rt[NPT][SN];

    auto load_slice_v = [&](auto vtag, int j0) {
        constexpr bool VEC = decltype(vtag)::value;
        const int j = j0 + scol;
#pragma unroll
        for (int s = 0; s < SB; ++s)
            load_query_raw<MODEL, VEC>(ph[s], pr[s], pw[s], pq[s], j, okb[s] ? klen : 0, half, qraw[s]);
#pragma unroll
        for (int s = 0; s < SN; ++s) {
            const int lim = okk[s] ? klen : 0;
            rt[0][s] = ld4_raw<VEC>(pt[s], j, lim);
            if constexpr (MODEL == KGE_ROTATE) rt[1][s] = ld4_raw<VEC>(pt[s] + half, j, lim);
        }
    };

    auto load_slice = [&](int j0, int) {  // one uniform branch per slice, none per load
        load_slice_v(std::integral_constant<bool, VEC4>{}, j0);
    };

    // the slice that load_slice(j0) requested: query rows formed, tails masked, written to LDS
    auto stage_slice_v = [&](auto vtag, int j0) {
        constexpr bool VEC = decltype(vtag)::value;
        const int j = j0 + scol;
#pragma unroll
        for (int q = 0; q < SB; ++q) {
            float4 q0, q1;
            combine_query<MODEL, VEC>(qraw[q], pa[q], j, okb[q] ? klen : 0, half, a.rsign, q0, q1);
            *reinterpret_cast<float4 *>(&sA[0][srow + 32 * q][scol]) = kScaled ? scale4(q0, kSgnScale) : q0;
            if constexpr (NPA == 2)
                *reinterpret_cast<float4 *>(&sA[1][srow + 32 * q][scol]) = kScaled ? scale4(q1, kSgnScale) : q1;
        }
#pragma unroll
        for (int q = 0; q < SN; ++q)
#pragma unroll
            for (int pl = 0; pl < NPT; ++pl) {
                const float4 v = mask4<VEC>(rt[pl][q], j, okk[q] ? klen : 0);
                *reinterpret_cast<float4 *>(&sT[pl][srow + 32 * q][scol]) = kScaled ? scale4(v, kSgnScale) : v;
            }
    };
    auto stage_slice = [&](int j0) {
        stage_slice_v(std::integral_constant<bool, VEC4>{}, j0);
    };

    float acc[RB][RK], cdot[RB][RK], acc2[RB][RK];
#pragma unroll
    for (int i = 0; i < RB; ++i)
#pragma unroll
        for (int k = 0; k < RK; ++k) acc[i][k] = 0.0f, cdot[i][k] = 0.0f, acc2[i][k] = 0.0f;

    const int nslice = (klen + kKD - 1) / kKD;
    int slice0 = 0, slice1 = nslice;  // this workgroup's share of the reduction axis
    if (a.ksplit > 1) {
        const int per = (nslice + a.ksplit - 1) / a.ksplit;
        slice0 = split * per;
        slice1 = slice0 + per < nslice ? slice0 + per : nslice;
    }
    // One sweep over the reduction axis.  `pass` is a compile-time tag: TransH's first sweep (the
    // w . t' dot products) and second sweep (the norm) get their own straight-line inner loops; as a
    // run-time value it put a branch around every pair of the micro-tile.
    auto sweep = [&](auto pass_tag) {
        constexpr int pass = decltype(pass_tag)::value;
        constexpr int kInnerUnroll = (MODEL == KGE_TRANSH || (MODEL == KGE_ROTATE && RB == 4)) ? 2 : kKD / 4;
        if (slice0 < slice1) load_slice(slice0 * kKD, pass);
#pragma unroll 1
        for (int s = slice0; s < slice1; ++s) {
            stage_slice(s * kKD);
            __syncthreads();
            if (s + 1 < slice1) load_slice((s + 1) * kKD, pass);
            __builtin_amdgcn_sched_barrier(0);  // (the requests go out before the compute, not after it)
            // (TransH keeps three sums per pair, RotatE two row planes: unrolled all the way, the hoisted LDS reads push the
            // 4 x 4 micro-tile over the register budget and twenty to fifty registers per lane go through
            // scratch memory every step)
#pragma unroll kInnerUnroll
            for (int i4 = 0; i4 < kKD / 4; ++i4) {
                float4 av[NPA][RB], tv[NPT][RK];
#pragma unroll
                for (int pl = 0; pl < NPA; ++pl)
#pragma unroll
                    for (int i = 0; i < RB; ++i)
                        av[pl][i] = *reinterpret_cast<const float4 *>(&sA[pl][ty + 16 * i][i4 * 4]);
#pragma unroll
                for (int pl = 0; pl < NPT; ++pl)
#pragma unroll
                    for (int k = 0; k < RK; ++k)
                        tv[pl][k] = *reinterpret_cast<const float4 *>(&sT[pl][tx + 16 * k][i4 * 4]);
#pragma unroll
                for (int i = 0; i < RB; ++i)
#pragma unroll
                    for (int k = 0; k < RK; ++k) {
                        const float4 a0 = av[0][i], a1 = av[NPA - 1][i];
                        const float4 t0 = tv[0][k], t1 = tv[NPT - 1][k];
                        if constexpr (MODEL == KGE_TRANSH && pass == 0) {
                            float &cc = cdot[i][k];
                            cc = fmaf(a1.x, t0.x, cc);
                            cc = fmaf(a1.y, t0.y, cc);
                            cc = fmaf(a1.z, t0.z, cc);
                            cc = fmaf(a1.w, t0.w, cc);
                        } else {
                            const float cc = cdot[i][k];
                            pair_elem<MODEL, P, SAVE>(acc[i][k], acc2[i][k], a0.x, a1.x, t0.x, t1.x, cc);
                            pair_elem<MODEL, P, SAVE>(acc[i][k], acc2[i][k], a0.y, a1.y, t0.y, t1.y, cc);
                            pair_elem<MODEL, P, SAVE>(acc[i][k], acc2[i][k], a0.z, a1.z, t0.z, t1.z, cc);
                            pair_elem<MODEL, P, SAVE>(acc[i][k], acc2[i][k], a0.w, a1.w, t0.w, t1.w, cc);
                        }
                    }
            }
            __syncthreads();
        }
    };
    if constexpr (MODEL == KGE_TRANSH) {
        // TransH, first sweep: c[b][k] = w_b . t'_k for the whole tile is a matrix product (normal
        // rows x negative rows), run on the matrix cores (v_mfma_f32_16x16x4_f32; operand layout
        // and k relabelling as in score_neg_mfma_kernel below).  Only the w and t' rows are staged.
        // The four waves tile the workgroup 2 x 2; the products then go through LDS into the
        // (ty + 16 i, tx + 16 k) layout of the second sweep's micro-tiles.
        constexpr int MB = RB / 2, NB = RK / 2;
        const int lane = tid & 63, wave = tid >> 6, fr = lane & 15, fg = lane >> 4;
        const int wrow = (wave >> 1) * (TB / 2), wcol = (wave & 1) * (TN / 2);
        v4f macc[MB][NB];
#pragma unroll
        for (int m = 0; m < MB; ++m)
#pragma unroll
            for (int n = 0; n < NB; ++n) macc[m][n] = v4f{0.0f, 0.0f, 0.0f, 0.0f};
        float4 rw[SB];
        auto load_w = [&](int j0) {  // one uniform branch per slice, none per load
            const int j = j0 + scol;
#pragma unroll
            for (int q = 0; q < SB; ++q) rw[q] = ld4_raw<VEC4>(pw[q], j, okb[q] ? d : 0);
#pragma unroll
            for (int q = 0; q < SN; ++q) rt[0][q] = ld4_raw<VEC4>(pt[q], j, okk[q] ? d : 0);
        };
        auto stage_w = [&](int j0) {  // (raw loads, masked when written: see load_slice_v)
            const int j = j0 + scol;
#pragma unroll
            for (int q = 0; q < SB; ++q) {
                const int lim = okb[q] ? d : 0;
                *reinterpret_cast<float4 *>(&sA[1][srow + 32 * q][scol]) = mask4<VEC4>(rw[q], j, lim);
            }
#pragma unroll
            for (int q = 0; q < SN; ++q) {
                const int lim = okk[q] ? d : 0;
                *reinterpret_cast<float4 *>(&sT[0][srow + 32 * q][scol]) = mask4<VEC4>(rt[0][q], j, lim);
            }
        };
        load_w(0);
#pragma unroll 1
        for (int s = 0; s < nslice; ++s) {
            stage_w(s * kKD);
            __syncthreads();
            if (s + 1 < nslice) load_w((s + 1) * kKD);
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int g = 0; g < kKD / 16; ++g) {
                float4 av[MB], tv[NB];
#pragma unroll
                for (int m = 0; m < MB; ++m)
                    av[m] = *reinterpret_cast<const float4 *>(&sA[1][wrow + 16 * m + fr][16 * g + 4 * fg]);
#pragma unroll
                for (int n = 0; n < NB; ++n)
                    tv[n] = *reinterpret_cast<const float4 *>(&sT[0][wcol + 16 * n + fr][16 * g + 4 * fg]);
#pragma unroll
                for (int e = 0; e < 4; ++e)
#pragma unroll
                    for (int m = 0; m < MB; ++m)
#pragma unroll
                        for (int n = 0; n < NB; ++n) {
                            const float x = e == 0 ? av[m].x : e == 1 ? av[m].y : e == 2 ? av[m].z : av[m].w;
                            const float y = e == 0 ? tv[n].x : e == 1 ? tv[n].y : e == 2 ? tv[n].z : tv[n].w;
                            macc[m][n] = __builtin_amdgcn_mfma_f32_16x16x4f32(x, y, macc[m][n], 0, 0, 0);
                        }
            }
            __syncthreads();
        }
        // D[i = 4 (l / 16) + v][j = l % 16] of block (m, n) -> sC[row][col] -> cdot of the micro-tiles
        float(*sC)[TN + 1] = reinterpret_cast<float(*)[TN + 1]>(dyn_smem);  // TB x (TN + 1) floats fit in plane 0 + 1 of sA
        static_assert(sizeof(float) * TB * (TN + 1) <= sizeof(float) * NPA * TB * kLDW + sizeof(float) * NPT * TN * kLDW,
                      "the product tile reuses the staging buffers");
#pragma unroll
        for (int m = 0; m < MB; ++m)
#pragma unroll
            for (int n = 0; n < NB; ++n)
#pragma unroll
                for (int v = 0; v < 4; ++v) sC[wrow + 16 * m + 4 * fg + v][wcol + 16 * n + fr] = macc[m][n][v];
        __syncthreads();
#pragma unroll
        for (int i = 0; i < RB; ++i)
#pragma unroll
            for (int k = 0; k < RK; ++k) cdot[i][k] = sC[ty + 16 * i][tx + 16 * k];
        __syncthreads();
        sweep(std::integral_constant<int, 1>{});
    } else {
        sweep(std::integral_constant<int, 0>{});
    }

#pragma unroll
    for (int i = 0; i < RB; ++i) {
        const int bl = bt0 + ty + 16 * i;
        if (bl >= a.C) continue;
        const int64_t rowoff = ((int64_t)c * a.C + bl) * a.N;
#pragma unroll
        for (int k = 0; k < RK; ++k) {
            const int kl = kt0 + tx + 16 * k;
            if (kl >= a.N) continue;
            float s = acc[i][k];
            if (a.ksplit > 1) {  // raw sum of this workgroup's slices; finished by score_neg_finish_kernel
                a.partial[(int64_t)split * a.plane + rowoff + kl] = s;
                continue;
            }
            if constexpr (kScaled) s *= kSgnUnscale, acc2[i][k] *= kSgnUnscale;
            if constexpr (MODEL == KGE_TRANSE || MODEL == KGE_TRANSH) s = P == 2 ? sqrtf(s) : s;
            if constexpr (MODEL == KGE_ROTATE) s = a.gamma - s;
            if constexpr (MODEL == KGE_TRANSF) s -= a.rsign * a.side_pos[(int64_t)c * a.C + bl];
            a.out[rowoff + kl] = s;
            if constexpr (MODEL == KGE_TRANSH && SAVE) {
                a.side_neg[rowoff + kl] = cdot[i][k];
                a.side_neg[a.plane + rowoff + kl] = P == 1 ? acc2[i][k] : (s > 0.0f ? acc2[i][k] / s : 0.0f);
            }
        }
    }
}

// DistMult / ComplEx: the pair scores of a tile are a plain matrix product, query rows (TB x d)
// times negative rows (TN x d) transposed, so the inner loop runs on the matrix cores
// (v_mfma_f32_16x16x4_f32, fp32 in, fp32 accumulate).  Staging is the same as above; the four
// waves tile the workgroup 2 x 2 and each owns (TB/2) x (TN/2) scores as 16 x 16 blocks.
// Operand layout: lane l supplies A[i = l % 16][k = l / 16] and B[k = l / 16][j = l % 16] and
// receives D[i = 4 * (l / 16) + v][j = l % 16], v = 0..3.  Inside 16 consecutive k the MFMA step
// s pairs lane group g = l / 16 with k = 4 g + s (any pairing works as long as both operands use
// it), so a lane's values for four steps are one 128-bit LDS read of its row.

template <int MODEL, int RB, int RK, bool VEC4>
__global__ __launch_bounds__(256, KGE_TILE_OCC) void score_neg_mfma_kernel(NegArgs a, FusedInsp fi)
{
    extern __shared__ __align__(16) char dyn_smem[];
    if (fused_insp_block(fi, reinterpret_cast<uint32_t *>(dyn_smem))) return;
    static_assert(MODEL == KGE_DISTMULT || MODEL == KGE_COMPLEX || MODEL == KGE_TRANSF || MODEL == KGE_RESCAL,
                  "dot-product scores only");
    if (a.pos_blocks > 0 && (int)blockIdx.x - fi.blocks >= a.tile_blocks) {  // the positives carried along
        if constexpr (MODEL == KGE_DISTMULT || MODEL == KGE_COMPLEX)
            score_pos_body<MODEL, 2, 4>(a.pos, nullptr, (int64_t)((int)blockIdx.x - fi.blocks - a.tile_blocks));
        return;
    }
    constexpr int TB = 16 * RB, TN = 16 * RK;
    constexpr int SB = TB / 32, SN = TN / 32;
    constexpr int MB = RB / 2, NB = RK / 2;  // 16 x 16 blocks per wave
    static_assert(TB % 32 == 0 && TN % 32 == 0, "tile rows are staged 32 at a time");

    float(*sA)[kLDW] = reinterpret_cast<float(*)[kLDW]>(dyn_smem);
    float(*sT)[kLDW] = reinterpret_cast<float(*)[kLDW]>(dyn_smem + sizeof(float) * TB * kLDW);

    const int tid = threadIdx.x;
    const int srow = tid >> 3, scol = (tid & 7) * 4;
    const int lane = tid & 63, wave = tid >> 6;
    const int fr = lane & 15, fg = lane >> 4;
    const int wrow = (wave >> 1) * (TB / 2), wcol = (wave & 1) * (TN / 2);
    int c, tile_y, tile_x;
    if (!xcd_tile(blockIdx.x - fi.blocks, (a.N + TN - 1) / TN, (a.C + TB - 1) / TB, a.n_chunks, c, tile_y, tile_x)) return;
    const int bt0 = tile_y * TB, kt0 = tile_x * TN;
    const int d = a.d, half = d >> 1;
    // (VEC4, 128-bit row loads, is a compile-time choice: as a run-time one the compiler merges the two
    // forms of the raw loads into the scalar one)

    const float *ph[SB], *pr[SB], *pq[SB];
    bool okb[SB];
#pragma unroll
    for (int s = 0; s < SB; ++s) {
        const int bl = bt0 + srow + 32 * s;
        okb[s] = bl < a.C;
        const int64_t b = (int64_t)c * a.C + (okb[s] ? bl : a.C - 1);
        ph[s] = a.ent + a.h[b] * (int64_t)d;
        pr[s] = a.rel + a.r[b] * (int64_t)a.rel_dim;
        pq[s] = MODEL == KGE_RESCAL ? a.query + b * (int64_t)d : nullptr;
    }
    const float *pt[SN];
    bool okk[SN];
#pragma unroll
    for (int s = 0; s < SN; ++s) {
        const int kl = kt0 + srow + 32 * s;
        okk[s] = kl < a.N;
        pt[s] = a.ent + a.neg[(int64_t)c * a.N + (okk[s] ? kl : a.N - 1)] * (int64_t)d;
    }

    // Raw operands of the next slice are in flight during the matrix-core work of this one; they are
    // combined into the query rows and masked when they are written to LDS (see score_neg_kernel).
    // (Two or four slices ahead measure the same: the launch is bound by its index chains and its
    // eight barrier pairs, not by the rows' latency.)
    constexpr int NRAW = query_raw_count<MODEL>();
    float4 qraw[SB][NRAW], rt[SN];
    auto load_slice = [&](int j0, float4 (&qr)[SB][NRAW], float4 (&tr)[SN]) {
        const int j = j0 + scol;
#pragma unroll
        for (int s = 0; s < SB; ++s) load_query_raw<MODEL, VEC4>(ph[s], pr[s], nullptr, pq[s], j, okb[s] ? d : 0, half, qr[s]);
#pragma unroll
        for (int s = 0; s < SN; ++s) tr[s] = ld4_raw<VEC4>(pt[s], j, okk[s] ? d : 0);
    };
    auto stage_slice = [&](int j0, const float4 (&qr)[SB][NRAW], const float4 (&tr)[SN]) {
        const int j = j0 + scol;
#pragma unroll
        for (int q = 0; q < SB; ++q) {
            float4 q0, q1;
            combine_query<MODEL, VEC4>(qr[q], 0.0f, j, okb[q] ? d : 0, half, a.rsign, q0, q1);
            *reinterpret_cast<float4 *>(&sA[srow + 32 * q][scol]) = q0;
        }
#pragma unroll
        for (int q = 0; q < SN; ++q)
            *reinterpret_cast<float4 *>(&sT[srow + 32 * q][scol]) = mask4<VEC4>(tr[q], j, okk[q] ? d : 0);
    };

    // two accumulators per block (one per half of the slice) keep consecutive MFMAs independent
    v4f acc[2][MB][NB];
#pragma unroll
    for (int g = 0; g < 2; ++g)
#pragma unroll
        for (int m = 0; m < MB; ++m)
#pragma unroll
            for (int n = 0; n < NB; ++n) acc[g][m][n] = v4f{0.0f, 0.0f, 0.0f, 0.0f};

    const int nslice = (d + kKD - 1) / kKD;
    load_slice(0, qraw, rt);
#pragma unroll 1
    for (int s = 0; s < nslice; ++s) {
        stage_slice(s * kKD, qraw, rt);
        __syncthreads();
        if (s + 1 < nslice) load_slice((s + 1) * kKD, qraw, rt);
        __builtin_amdgcn_sched_barrier(0);  // (the requests go out before the matrix-core work, not after it)
#pragma unroll
        for (int g = 0; g < kKD / 16; ++g) {
            float4 av[MB], tv[NB];
#pragma unroll
            for (int m = 0; m < MB; ++m)
                av[m] = *reinterpret_cast<const float4 *>(&sA[wrow + 16 * m + fr][16 * g + 4 * fg]);
#pragma unroll
            for (int n = 0; n < NB; ++n)
                tv[n] = *reinterpret_cast<const float4 *>(&sT[wcol + 16 * n + fr][16 * g + 4 * fg]);
#pragma unroll
            for (int e = 0; e < 4; ++e)
#pragma unroll
                for (int m = 0; m < MB; ++m)
#pragma unroll
                    for (int n = 0; n < NB; ++n) {
                        const float x = e == 0 ? av[m].x : e == 1 ? av[m].y : e == 2 ? av[m].z : av[m].w;
                        const float y = e == 0 ? tv[n].x : e == 1 ? tv[n].y : e == 2 ? tv[n].z : tv[n].w;
                        acc[g & 1][m][n] = __builtin_amdgcn_mfma_f32_16x16x4f32(x, y, acc[g & 1][m][n], 0, 0, 0);
                    }
        }
        __syncthreads();
    }

#pragma unroll
    for (int m = 0; m < MB; ++m)
#pragma unroll
        for (int v = 0; v < 4; ++v) {
            const int bl = bt0 + wrow + 16 * m + 4 * fg + v;
            if (bl >= a.C) continue;
            const int64_t rowoff = ((int64_t)c * a.C + bl) * a.N;
            float shift = 0.0f;  // TransF: the per-positive constant -r.h (+r.t with head negatives)
            if constexpr (MODEL == KGE_TRANSF) shift = -a.rsign * a.side_pos[(int64_t)c * a.C + bl];
#pragma unroll
            for (int n = 0; n < NB; ++n) {
                const int kl = kt0 + wcol + 16 * n + fr;
                if (kl < a.N) a.out[rowoff + kl] = (acc[0][m][n][v] + acc[1][m][n][v]) + shift;
            }
        }
}

// LDS bytes of a launch: the tile's staging buffers, or what the inspector workgroups need if more
static size_t neg_lds(int planes, int TB, int TN, int planes_t, const FusedInsp &fi)
{
    const size_t own = sizeof(float) * kLDW * ((size_t)planes * TB + (size_t)planes_t * TN);
    return fi.blocks > 0 && (size_t)fi.lds_bytes > own ? (size_t)fi.lds_bytes : own;
}

// Adds the partial planes of a split reduction axis and finishes the scores.
template <int MODEL, int P>
__global__ __launch_bounds__(256) void score_neg_finish_kernel(const float *partial, int ksplit, int64_t plane, float gamma,
                                                               float *out)
{
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= plane) return;
    float s = partial[i];
    for (int q = 1; q < ksplit; ++q) s += partial[(int64_t)q * plane + i];
    if constexpr (MODEL == KGE_TRANSE) s = P == 2 ? sqrtf(s) : s;
    if constexpr (MODEL == KGE_ROTATE) s = gamma - s;
    out[i] = s;
}

// Workgroups per tile along the reduction axis.  A batch whose 32 x 32 tiles leave one or two
// workgroups per CU runs every instruction at its full latency (a single wave per SIMD has nobody
// to interleave with): splitting the row over up to four workgroups multiplies the waves.  Only
// for the models whose pair score is one plain sum over the row (TransE, RotatE).
int neg_ksplit(const kge_tables *tab, const kge_batch *bat)
{
    if (!bat->neg || bat->chunk <= 0 || (tab->model != KGE_TRANSE && tab->model != KGE_ROTATE)) return 1;
    const int64_t n_chunks = bat->batch / bat->chunk;
    if (n_chunks <= 0 || ceil_div(bat->chunk, 64) * ceil_div(bat->n_neg, 64) * n_chunks >= 1024) return 1;  // (64 x 64 tiles)
    const int64_t tiles = xcd_grid(ceil_div(bat->n_neg, 32), ceil_div(bat->chunk, 32), n_chunks);
    const int64_t klen = tab->model == KGE_ROTATE ? tab->dim / 2 : tab->dim;
    const int64_t nslice = ceil_div(klen, kKD);
    int64_t s = 1024 / tiles;
    s = s > 4 ? 4 : s;
    while (s > 1 && nslice / s < 4) --s;
    return s < 1 ? 1 : (int)s;
}

size_t neg_split_workspace(const kge_tables *tab, const kge_batch *bat)
{
    const int s = neg_ksplit(tab, bat);
    return s > 1 ? sizeof(float) * (size_t)s * (size_t)(bat->batch * bat->n_neg) : 0;
}

// one launch, the 128-bit-load form of the kernel where the rows allow it
template <typename K>
static void launch_neg_k(K kernel, dim3 grid, size_t lds, hipStream_t st, const NegArgs &a, const FusedInsp &fi)
{
    hipLaunchKernelGGL(kernel, grid, dim3(256), lds, st, a, fi);
}
#define NEG_LAUNCH(KERNEL, ...)                                                    \
    (a.vec ? launch_neg_k(KERNEL<__VA_ARGS__, true>, grid, lds, st, a, fi)         \
           : launch_neg_k(KERNEL<__VA_ARGS__, false>, grid, lds, st, a, fi))
#define NEG_LAUNCH_VEC(KERNEL, ...) launch_neg_k(KERNEL<__VA_ARGS__, true>, grid, lds, st, a, fi)

template <int MODEL, int P>
static int launch_neg_mp(const NegArgs &a_in, int64_t n_chunks, bool dot_valu, const FusedInsp &fi, hipStream_t st)
{
    NegArgs a = a_in;
    constexpr int NPA = (MODEL == KGE_ROTATE || MODEL == KGE_TRANSH) ? 2 : 1, NPT = MODEL == KGE_ROTATE ? 2 : 1;
    const int64_t big_tiles = ceil_div(a.C, 64) * ceil_div(a.N, 64) * n_chunks;
    // Small tiles up to about 1024 big tiles: more waves to hide latency (32x32 is ~20 % faster than
    // 64x64 on a 256-big-tile workload with the vector-ALU loop; the matrix-core loop, whose
    // launches are bound by the rows its workgroups pull from L2, does best with 32x64).  The
    // inspector workgroups that share the machine with these launches raise their wave priority.
    constexpr bool kDotModel = MODEL == KGE_DISTMULT || MODEL == KGE_COMPLEX || MODEL == KGE_TRANSF || MODEL == KGE_RESCAL;
    // Rows without 128-bit loads (dim % 4 != 0, unaligned tables) take the 32x32 tile whatever the size:
    // only that tile is compiled in the scalar-load form.
    const int tile = !a.vec ? 2 : big_tiles >= 1024 ? 4 : (kDotModel && !dot_valu ? 3 : 2);  // 2: 32x32, 3: 32x64, 4: 64x64
    const int TB = tile == 4 ? 64 : 32, TN = tile == 2 ? 32 : 64;
    // (workgroups that score the positives, if the launch carries them, follow the tiles')
    const unsigned tile_blocks = xcd_grid(ceil_div(a.N, TN), ceil_div(a.C, TB), n_chunks) * (unsigned)(a.ksplit > 1 ? a.ksplit : 1);
    a.tile_blocks = (int)tile_blocks;
    const dim3 grid(tile_blocks + (unsigned)fi.blocks + (unsigned)a.pos_blocks);
    if constexpr (kDotModel) {
        if (!dot_valu) {
            const size_t lds = neg_lds(1, TB, TN, 1, fi);
            if (tile == 4) NEG_LAUNCH_VEC(score_neg_mfma_kernel, MODEL, 4, 4);
            else if (tile == 3) NEG_LAUNCH_VEC(score_neg_mfma_kernel, MODEL, 2, 4);
            else NEG_LAUNCH(score_neg_mfma_kernel, MODEL, 2, 2);
            KGE_CHECK_LAUNCH();
            return KGE_OK;
        }
    }
    const size_t lds = neg_lds(NPA, TB, TN, NPT, fi);
    const bool save = MODEL == KGE_TRANSH && a.side_neg;
    if (a.ksplit > 1) {  // (neg_ksplit: 32 x 32 tiles of TransE / RotatE)
        if constexpr (MODEL == KGE_TRANSE || MODEL == KGE_ROTATE) {
            NEG_LAUNCH(score_neg_kernel, MODEL, P, 2, 2, false);
            hipLaunchKernelGGL((score_neg_finish_kernel<MODEL, P>), dim3((unsigned)ceil_div(a.plane, 256)), dim3(256), 0, st,
                               a.partial, a.ksplit, a.plane, a.gamma, a.out);
            KGE_CHECK_LAUNCH();
            return KGE_OK;
        }
        return KGE_EINVAL;
    }
    if (tile == 3) {  // 32 positives x 64 negatives
        if (save) NEG_LAUNCH_VEC(score_neg_kernel, MODEL, P, 2, 4, true);
        else NEG_LAUNCH_VEC(score_neg_kernel, MODEL, P, 2, 4, false);
    } else if (tile == 4) {
        if (save) NEG_LAUNCH_VEC(score_neg_kernel, MODEL, P, 4, 4, true);
        else NEG_LAUNCH_VEC(score_neg_kernel, MODEL, P, 4, 4, false);
    } else {
        if (save) NEG_LAUNCH(score_neg_kernel, MODEL, P, 2, 2, true);
        else NEG_LAUNCH(score_neg_kernel, MODEL, P, 2, 2, false);
    }
    KGE_CHECK_LAUNCH();
    return KGE_OK;
}

// True if the shared-negative launch of this batch can score the positives as well (carry_pos of
// launch_score_neg): TransE, or DistMult / ComplEx on the matrix-core tiles, with 128-bit row loads
// and no inspector workgroups in the launch (these models' tiles do not read what the positives'
// kernel writes).
bool score_neg_carries_positives(const kge_tables *tab, const kge_batch *bat)
{
    const bool dot = (tab->model == KGE_DISTMULT || tab->model == KGE_COMPLEX) && !pair_sums_valu(tab);
    return (dot || tab->model == KGE_TRANSE) && bat->neg && bat->batch > 0 && !bat->fuse_inspection && rows_vectorizable(tab) &&
           ceil_div(bat->batch, kPosWaves) < (1 << 30);
}

int launch_score_neg(const kge_tables *tab, const kge_batch *bat, const float *side_pos, const float *query,
                     float *out, float *side_neg, const FusedInsp *fused, void *workspace, size_t workspace_bytes,
                     hipStream_t st, float *carry_pos)
{
    const FusedInsp fi = fused ? *fused : FusedInsp{};
    if (bat->batch == 0) return KGE_OK;
    if (carry_pos && (fused || !score_neg_carries_positives(tab, bat))) return KGE_EINVAL;
    const int64_t n_chunks = bat->batch / bat->chunk;
    if (n_chunks >= (1 << 24) || bat->chunk >= (1 << 30) || bat->n_neg >= (1 << 30)) return KGE_ESHAPE;
    const bool vec = rows_vectorizable(tab);
    const bool head = bat->neg_mode == KGE_NEG_HEAD;
    NegArgs a{tab->ent, tab->rel, tab->aux, head ? bat->t : bat->h, bat->r, bat->neg, side_pos, query, out, side_neg,
              bat->batch * bat->n_neg, (int)bat->chunk, (int)bat->n_neg, (int)tab->dim, (int)tab->rel_dim, tab->gamma,
              vec ? 1 : 0, (int)n_chunks, head ? -1.0f : 1.0f, 1, nullptr, PosArgs{}, 0, 0};
    if (carry_pos) {
        a.pos = PosArgs{tab->ent, tab->rel, tab->aux, bat->h, bat->r, bat->t, bat->batch, (int)tab->dim, (int)tab->rel_dim,
                        tab->gamma, carry_pos, nullptr, nullptr, 0};
        a.pos_blocks = (int)ceil_div(bat->batch, kPosWaves);
    }
    // the reduction axis is split when the caller's workspace has room for the partial planes
    const int ksplit = neg_ksplit(tab, bat);
    if (ksplit > 1 && workspace && workspace_bytes >= neg_split_workspace(tab, bat) && aligned16(workspace))
        a.ksplit = ksplit, a.partial = static_cast<float *>(workspace);
    const int p = tab->norm_p;
    const bool dv = pair_sums_valu(tab);
    switch (tab->model) {
    case KGE_TRANSE:
        return p == 1 ? launch_neg_mp<KGE_TRANSE, 1>(a, n_chunks, dv, fi, st)
                      : launch_neg_mp<KGE_TRANSE, 2>(a, n_chunks, dv, fi, st);
    case KGE_TRANSH:
        return p == 1 ? launch_neg_mp<KGE_TRANSH, 1>(a, n_chunks, dv, fi, st)
                      : launch_neg_mp<KGE_TRANSH, 2>(a, n_chunks, dv, fi, st);
    case KGE_DISTMULT: return launch_neg_mp<KGE_DISTMULT, 2>(a, n_chunks, dv, fi, st);
    case KGE_COMPLEX: return launch_neg_mp<KGE_COMPLEX, 2>(a, n_chunks, dv, fi, st);
    case KGE_ROTATE: return launch_neg_mp<KGE_ROTATE, 2>(a, n_chunks, dv, fi, st);
    case KGE_TRANSF: return launch_neg_mp<KGE_TRANSF, 2>(a, n_chunks, dv, fi, st);
    case KGE_RESCAL:  // a dot-product tile over the projected rows: E[h] Proj[r] against replaced tails,
                      // Proj[r] E[t] against replaced heads
        if (!query) return KGE_EUNSUPPORTED;
        return launch_neg_mp<KGE_RESCAL, 2>(a, n_chunks, dv, fi, st);
    default: return KGE_EUNSUPPORTED;  // TransR: its own grouped path
    }
}

}  // namespace kge
