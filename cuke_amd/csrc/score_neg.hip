// Shared-negative forward: every positive of a chunk against the chunk's N
// negative tails (layout of apps/examples/examples.py:1404-1444, which the
// reference only ever lowers to serial CPU loops).
//
// One workgroup owns a (TB positives x TN negatives) tile of one chunk.  The
// "query" rows a_b = f(h_b, r_b) are formed while staging (the gathers of h and r
// are fused into the staging loads) and the negative rows are gathered straight
// into LDS, KD floats of the row at a time; each thread then accumulates an
// RB x RK block of pair scores from LDS with 128-bit reads.  All arithmetic is
// fp32 VALU; no matrix cores.
#include <stdlib.h>

#include "common.hpp"

namespace kge {

struct NegArgs {
    const float *ent, *rel, *aux;
    const int64_t *h, *r, *neg;
    const float *side_pos;  // TransH: w_b . h_b
    float *out;             // [B, N]
    float *side_neg;        // TransH: w_b . t'_k  [B, N] (optional)
    int C, N, d, rel_dim;
    float gamma;
    int vec;
};

constexpr int kKD = 32;        // floats of each row staged per step
constexpr int kLDW = kKD + 4;  // LDS row pitch: +4 floats keeps 128-bit reads of
                               // 8 consecutive rows on distinct banks

__device__ __forceinline__ float4 ld4(const float *p, int j, int lim, bool vec)
{
    if (vec) return j < lim ? *reinterpret_cast<const float4 *>(p + j) : make_float4(0, 0, 0, 0);
    float4 q;
    q.x = j + 0 < lim ? p[j + 0] : 0.0f;
    q.y = j + 1 < lim ? p[j + 1] : 0.0f;
    q.z = j + 2 < lim ? p[j + 2] : 0.0f;
    q.w = j + 3 < lim ? p[j + 3] : 0.0f;
    return q;
}

__device__ __forceinline__ float4 zero4() { return make_float4(0.f, 0.f, 0.f, 0.f); }

__device__ __forceinline__ float4 mul4(float4 p, float4 q)
{
    return make_float4(p.x * q.x, p.y * q.y, p.z * q.z, p.w * q.w);
}
__device__ __forceinline__ float4 add4(float4 p, float4 q)
{
    return make_float4(p.x + q.x, p.y + q.y, p.z + q.z, p.w + q.w);
}

// One element of the pair update, per model.
template <int MODEL, int P>
__device__ __forceinline__ void pair_elem(float &acc, float a0, float a1, float t0, float t1, float c)
{
    if constexpr (MODEL == KGE_DISTMULT || MODEL == KGE_COMPLEX) {
        acc = fmaf(a0, t0, acc);
    } else if constexpr (MODEL == KGE_TRANSE) {
        const float u = a0 - t0;
        if constexpr (P == 1) acc += fabsf(u);
        else acc = fmaf(u, u, acc);
    } else if constexpr (MODEL == KGE_TRANSH) {
        // a0 = h + r - (w.h) w, a1 = w, c = w . t'
        const float u = fmaf(c, a1, a0 - t0);
        if constexpr (P == 1) acc += fabsf(u);
        else acc = fmaf(u, u, acc);
    } else if constexpr (MODEL == KGE_ROTATE) {
        const float ur = a0 - t0, ui = a1 - t1;
        acc += __builtin_amdgcn_sqrtf(fmaf(ur, ur, ui * ui));
    }
}

template <int MODEL, int P, int RB, int RK>
__global__ __launch_bounds__(256) void score_neg_kernel(NegArgs a)
{
    constexpr int TB = 16 * RB, TN = 16 * RK;
    constexpr int NPA = (MODEL == KGE_ROTATE || MODEL == KGE_TRANSH) ? 2 : 1;
    constexpr int NPT = MODEL == KGE_ROTATE ? 2 : 1;
    constexpr int SB = TB / 32, SN = TN / 32;  // float4 per thread per plane per step
    constexpr int NPASS = MODEL == KGE_TRANSH ? 2 : 1;
    static_assert(TB % 32 == 0 && TN % 32 == 0, "tile rows are staged 32 at a time");

    __shared__ __align__(16) float sA[NPA][TB][kLDW];
    __shared__ __align__(16) float sT[NPT][TN][kLDW];

    const int tid = threadIdx.x, tx = tid & 15, ty = tid >> 4;
    const int srow = tid >> 3, scol = (tid & 7) * 4;
    const int c = blockIdx.z, bt0 = blockIdx.y * TB, kt0 = blockIdx.x * TN;
    const int d = a.d, half = d >> 1;
    const int klen = MODEL == KGE_ROTATE ? half : d;
    const bool vec = a.vec != 0;

    // rows this thread stages
    const float *ph[SB], *pr[SB], *pw[SB];
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
    }
    const float *pt[SN];
    bool okk[SN];
#pragma unroll
    for (int s = 0; s < SN; ++s) {
        const int kl = kt0 + srow + 32 * s;
        okk[s] = kl < a.N;
        pt[s] = a.ent + a.neg[(int64_t)c * a.N + (okk[s] ? kl : a.N - 1)] * (int64_t)d;
    }

    float4 ra[NPA][SB], rt[NPT][SN];

    auto load_slice = [&](int j0, int pass) {
        const int j = j0 + scol;
#pragma unroll
        for (int s = 0; s < SB; ++s) {
            const int lim = okb[s] ? klen : 0;
            if constexpr (MODEL == KGE_DISTMULT) {
                const float4 vh = ld4(ph[s], j, lim, vec), vr = ld4(pr[s], j, lim, vec);
                ra[0][s] = mul4(vh, vr);
            } else if constexpr (MODEL == KGE_TRANSE) {
                const float4 vh = ld4(ph[s], j, lim, vec), vr = ld4(pr[s], j, lim, vec);
                ra[0][s] = add4(vh, vr);
            } else if constexpr (MODEL == KGE_COMPLEX) {
                // flat index j over [re | im]: a_re = hr*rr - hi*ri, a_im = hr*ri + hi*rr
                float q[4];
                if (vec) {  // half % 4 == 0: the four elements sit on one side of the split
                    const bool re = j < half;
                    const int i = re ? j : j - half;
                    const int l2 = lim ? half : 0;
                    const float4 hr = ld4(ph[s], i, l2, true), hi = ld4(ph[s] + half, i, l2, true);
                    const float4 rr = ld4(pr[s], i, l2, true), ri = ld4(pr[s] + half, i, l2, true);
                    q[0] = re ? hr.x * rr.x - hi.x * ri.x : hr.x * ri.x + hi.x * rr.x;
                    q[1] = re ? hr.y * rr.y - hi.y * ri.y : hr.y * ri.y + hi.y * rr.y;
                    q[2] = re ? hr.z * rr.z - hi.z * ri.z : hr.z * ri.z + hi.z * rr.z;
                    q[3] = re ? hr.w * rr.w - hi.w * ri.w : hr.w * ri.w + hi.w * rr.w;
                } else
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const int jj = j + e;
                    if (jj < lim) {
                        const int i = jj < half ? jj : jj - half;
                        const float hr = ph[s][i], hi = ph[s][i + half];
                        const float rr = pr[s][i], ri = pr[s][i + half];
                        q[e] = jj < half ? hr * rr - hi * ri : hr * ri + hi * rr;
                    } else {
                        q[e] = 0.0f;
                    }
                }
                ra[0][s] = make_float4(q[0], q[1], q[2], q[3]);
            } else if constexpr (MODEL == KGE_ROTATE) {
                const float4 hr = ld4(ph[s], j, lim, vec), hi = ld4(ph[s] + half, j, lim, vec);
                const float4 th = ld4(pr[s], j, lim, vec);
                float4 sn, cs;
                sincosf(th.x, &sn.x, &cs.x);
                sincosf(th.y, &sn.y, &cs.y);
                sincosf(th.z, &sn.z, &cs.z);
                sincosf(th.w, &sn.w, &cs.w);
                ra[0][s] = make_float4(hr.x * cs.x - hi.x * sn.x, hr.y * cs.y - hi.y * sn.y,
                                       hr.z * cs.z - hi.z * sn.z, hr.w * cs.w - hi.w * sn.w);
                ra[1][s] = make_float4(hr.x * sn.x + hi.x * cs.x, hr.y * sn.y + hi.y * cs.y,
                                       hr.z * sn.z + hi.z * cs.z, hr.w * sn.w + hi.w * cs.w);
            } else if constexpr (MODEL == KGE_TRANSH) {
                const float4 vw = ld4(pw[s], j, lim, vec);
                ra[1][s] = vw;
                if (pass == 1) {
                    const float4 vh = ld4(ph[s], j, lim, vec), vr = ld4(pr[s], j, lim, vec);
                    const float al = pa[s];
                    ra[0][s] = make_float4((vh.x + vr.x) - al * vw.x, (vh.y + vr.y) - al * vw.y,
                                           (vh.z + vr.z) - al * vw.z, (vh.w + vr.w) - al * vw.w);
                } else {
                    ra[0][s] = zero4();
                }
            }
        }
#pragma unroll
        for (int s = 0; s < SN; ++s) {
            const int lim = okk[s] ? klen : 0;
            rt[0][s] = ld4(pt[s], j, lim, vec);
            if constexpr (MODEL == KGE_ROTATE) rt[1][s] = ld4(pt[s] + half, j, lim, vec);
        }
    };

    float acc[RB][RK], cdot[RB][RK];
#pragma unroll
    for (int i = 0; i < RB; ++i)
#pragma unroll
        for (int k = 0; k < RK; ++k) acc[i][k] = 0.0f, cdot[i][k] = 0.0f;

    const int nslice = (klen + kKD - 1) / kKD;
#pragma unroll 1
    for (int pass = 0; pass < NPASS; ++pass) {
        load_slice(0, pass);
#pragma unroll 1
        for (int s = 0; s < nslice; ++s) {
#pragma unroll
            for (int q = 0; q < SB; ++q)
#pragma unroll
                for (int pl = 0; pl < NPA; ++pl)
                    *reinterpret_cast<float4 *>(&sA[pl][srow + 32 * q][scol]) = ra[pl][q];
#pragma unroll
            for (int q = 0; q < SN; ++q)
#pragma unroll
                for (int pl = 0; pl < NPT; ++pl)
                    *reinterpret_cast<float4 *>(&sT[pl][srow + 32 * q][scol]) = rt[pl][q];
            __syncthreads();
            if (s + 1 < nslice) load_slice((s + 1) * kKD, pass);
#pragma unroll
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
                        if (MODEL == KGE_TRANSH && pass == 0) {
                            float &cc = cdot[i][k];
                            cc = fmaf(a1.x, t0.x, cc);
                            cc = fmaf(a1.y, t0.y, cc);
                            cc = fmaf(a1.z, t0.z, cc);
                            cc = fmaf(a1.w, t0.w, cc);
                        } else {
                            const float cc = cdot[i][k];
                            pair_elem<MODEL, P>(acc[i][k], a0.x, a1.x, t0.x, t1.x, cc);
                            pair_elem<MODEL, P>(acc[i][k], a0.y, a1.y, t0.y, t1.y, cc);
                            pair_elem<MODEL, P>(acc[i][k], a0.z, a1.z, t0.z, t1.z, cc);
                            pair_elem<MODEL, P>(acc[i][k], a0.w, a1.w, t0.w, t1.w, cc);
                        }
                    }
            }
            __syncthreads();
        }
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
            if constexpr (MODEL == KGE_TRANSE || MODEL == KGE_TRANSH) s = P == 2 ? sqrtf(s) : s;
            if constexpr (MODEL == KGE_ROTATE) s = a.gamma - s;
            a.out[rowoff + kl] = s;
            if constexpr (MODEL == KGE_TRANSH)
                if (a.side_neg) a.side_neg[rowoff + kl] = cdot[i][k];
        }
    }
}

// 0: choose by size, 2: 32x32 tiles, 4: 64x64 tiles (development knob)
static int neg_tile_override()
{
    static const int v = [] {
        const char *e = getenv("KGE_NEG_TILE");
        return e ? atoi(e) : 0;
    }();
    return v;
}

template <int MODEL, int P>
static int launch_neg_mp(const NegArgs &a, int64_t n_chunks, hipStream_t st)
{
    const int64_t big_tiles = ceil_div(a.C, 64) * ceil_div(a.N, 64) * n_chunks;
    int tile = neg_tile_override();
    if (tile != 2 && tile != 4) tile = big_tiles >= 1024 ? 4 : 2;
    if (tile == 4) {
        const dim3 grid((unsigned)ceil_div(a.N, 64), (unsigned)ceil_div(a.C, 64), (unsigned)n_chunks);
        hipLaunchKernelGGL((score_neg_kernel<MODEL, P, 4, 4>), grid, dim3(256), 0, st, a);
    } else {
        const dim3 grid((unsigned)ceil_div(a.N, 32), (unsigned)ceil_div(a.C, 32), (unsigned)n_chunks);
        hipLaunchKernelGGL((score_neg_kernel<MODEL, P, 2, 2>), grid, dim3(256), 0, st, a);
    }
    KGE_CHECK_LAUNCH();
    return KGE_OK;
}

int launch_score_neg(const kge_tables *tab, const kge_batch *bat, const float *side_pos, float *out,
                     float *side_neg, hipStream_t st)
{
    if (bat->batch == 0) return KGE_OK;
    const int64_t n_chunks = bat->batch / bat->chunk;
    if (n_chunks > 65535 || bat->chunk >= (1 << 30) || bat->n_neg >= (1 << 30)) return KGE_ESHAPE;
    const bool complex_rows = tab->model == KGE_COMPLEX || tab->model == KGE_ROTATE;
    const bool vec = tab->dim % (complex_rows ? 8 : 4) == 0 && aligned16(tab->ent) &&
                     aligned16(tab->rel) && (!tab->aux || aligned16(tab->aux));
    NegArgs a{tab->ent, tab->rel, tab->aux, bat->h, bat->r, bat->neg, side_pos, out, side_neg,
              (int)bat->chunk, (int)bat->n_neg, (int)tab->dim, (int)tab->rel_dim, tab->gamma, vec ? 1 : 0};
    const int p = tab->norm_p;
    switch (tab->model) {
    case KGE_TRANSE:
        return p == 1 ? launch_neg_mp<KGE_TRANSE, 1>(a, n_chunks, st)
                      : launch_neg_mp<KGE_TRANSE, 2>(a, n_chunks, st);
    case KGE_TRANSH:
        return p == 1 ? launch_neg_mp<KGE_TRANSH, 1>(a, n_chunks, st)
                      : launch_neg_mp<KGE_TRANSH, 2>(a, n_chunks, st);
    case KGE_DISTMULT: return launch_neg_mp<KGE_DISTMULT, 2>(a, n_chunks, st);
    case KGE_COMPLEX: return launch_neg_mp<KGE_COMPLEX, 2>(a, n_chunks, st);
    case KGE_ROTATE: return launch_neg_mp<KGE_ROTATE, 2>(a, n_chunks, st);
    default: return KGE_EUNSUPPORTED;  // TransR / TransF / RESCAL: positives only
    }
}

}  // namespace kge
