// Backward of the score path: per-occurrence gradient rows, then an atomic-free
// segmented reduction to one row per distinct table row.
//
// The reference only prints per-triple dense gradient kernels (apps/kge/kge.py:393-515)
// and never scatters or reduces them; the gradients here are derived from the forward
// definitions (apps/kge/kge.py:273-390 and the DistMult / ComplEx / RotatE forms).
//
//   1. bwd_tile_kernel, owner = positives: G[b,:] = sum_k dneg[b,k] * d score(b,k) / d a_b
//   2. bwd_tile_kernel, owner = negatives: gradient row of every negative occurrence
//   3. bwd_pos_kernel: one wave per positive; chains G through a_b = f(h, r) and adds
//      the positive triple's own term; writes the h / t / r (/ w) occurrence rows
//   4. seg_reduce: occurrence rows are summed per distinct id in sorted order
//      (inspection perm / seg_offsets); every output row is written exactly once.
#include <type_traits>

#include "inspector_mid.hpp"
#include "seg_reduce.hpp"
#include "tile_common.hpp"

namespace kge {

typedef float v4f __attribute__((ext_vector_type(4)));

// ---------------------------------------------------------------------------------------
// 1 + 2: tile kernel.  "Owners" keep their slice of the row in registers and accumulate
// over all "loopers" of the chunk, which stream through LDS together with the
// per-(owner, looper) coefficients.
// ---------------------------------------------------------------------------------------
// The positive chain of the dot-product models, one element: G is the gradient with respect to the query
// row a = f(kept entity, relation) summed over the chunk's negatives, g the positive's own upstream
// gradient.  "kept" is the side of the positive the negatives do not replace (the head; the tail with
// head negatives), "other" the side they do.  Shared by the per-positive kernel and the tile kernel's
// epilogue, so both produce the same bits.
__device__ __forceinline__ void distmult_chain(float g, float k, float o, float r, float G, float &dk, float &dr, float &dother)
{
    const float Q = fmaf(g, o, G);  // a = k * r, score = a . other
    dk = r * Q;
    dr = k * Q;
    dother = g * (k * r);
}

// ComplEx: Re<h, r, conj t>.  Tail negatives: a = h o r;  head negatives: a = conj(r) o t.
template <bool HEAD>
__device__ __forceinline__ void complex_chain(float g, float kr, float ki, float or_, float oi, float qr, float qi, float Gr, float Gi,
                                              float &dkr, float &dki, float &drr, float &dri, float &dor, float &doi)
{
    const float Qr = fmaf(g, or_, Gr), Qi = fmaf(g, oi, Gi);
    if constexpr (HEAD) {
        dkr = fmaf(Qr, qr, -(Qi * qi));
        dki = fmaf(Qi, qr, Qr * qi);
        drr = fmaf(Qr, kr, Qi * ki);
        dri = fmaf(Qr, ki, -(Qi * kr));
        dor = g * fmaf(qr, kr, qi * ki);
        doi = g * fmaf(qr, ki, -(qi * kr));
    } else {
        dkr = fmaf(Qr, qr, Qi * qi);
        dki = fmaf(Qi, qr, -(Qr * qi));
        drr = fmaf(Qr, kr, Qi * ki);
        dri = fmaf(Qi, kr, -(Qr * ki));
        dor = g * fmaf(kr, qr, -(ki * qi));
        doi = g * fmaf(kr, qi, ki * qr);
    }
}

struct TileArgs {
    const float *ent, *rel, *aux;
    const int64_t *h, *r, *neg;
    const float *dneg;      // [B, N] upstream gradient
    const float *sneg;      // [B, N] forward scores (L2 normalisation)
    const float *side_pos;  // TransH: w.h per positive
    const float *side_neg;  // TransH: [2, B, N]
    const float *query;     // RotatE: rotated heads [B, d] saved by the forward pass; RESCAL: projected rows E[h] Proj[r]; else null
    float *out0, *out1;
    int64_t plane;  // B * N
    int C, N, d, rel_dim, vec, vecn, n_chunks;
    float rsign;    // +1: negatives replace the tail; -1: the head (h then holds the tails; see load_query)
    // Positive chain in the epilogue (DistMult / ComplEx on the matrix-core tiles, 128-bit rows, nothing
    // riding along): the workgroup that owns 64 positives x 64 columns holds the COMPLETE sum G over the
    // chunk's negatives for them, so it chains G through the query, adds the positive triple's own term and
    // writes the occurrence rows of both entities and of the relation itself.  No G rows go to memory and
    // come back, and no per-positive kernel runs.  chain == 0: G rows are written (out0) as for the other models.
    int chain;
    const int64_t *other;        // the positives' replaced side (tails; heads with head negatives)
    const float *dpos;           // [B] or null
    float *occ_k, *occ_o, *occ_r;  // occurrence rows [B, d] of the kept side, the replaced side, and [B, rel_dim]
};

constexpr int kTI = 64;       // columns of the row per workgroup
// Looper rows staged per step.  The 64-owner TransH tile holds two owner planes, two accumulator
// planes and three coefficient planes; with 32-row steps its prefetch registers spill (about 50
// registers per lane go through scratch memory every step: same speed, three times the memory
// traffic), with 16-row steps everything stays in registers.
template <int MODEL, int RO>
constexpr int looper_rows() { return MODEL == KGE_TRANSH && RO == 4 ? 16 : 32; }
constexpr int kLP = kTI + 4;  // LDS pitch of a staged row

template <int MODEL, bool OWNER_POS, int RO>
struct TileShape {
    static constexpr bool kRot = MODEL == KGE_ROTATE, kTH = MODEL == KGE_TRANSH;
    static constexpr int TO = 16 * RO;
    static constexpr int NPL = (kRot || (kTH && !OWNER_POS)) ? 2 : 1;
    static constexpr int NC = kTH ? 3 : 1;
    static constexpr int PG = TO + 4;
    static constexpr int kKL = looper_rows<MODEL, RO>();
    static constexpr int kLdsFloats = NPL * kKL * kLP + NC * kKL * PG;
};

// Width of the narrow last column tile: klen % 64 when that is between 1 and 16, else 0 (rows are
// then covered by 64-column tiles alone).
__host__ __device__ inline int narrow_cols(int klen)
{
    const int rem = klen % kTI;
    return rem > 0 && rem <= 16 ? rem : 0;
}

// NARROW: the tile covers the last 16 columns of rows whose width leaves a remainder of at most 16
// over the 64-column tiles.  A 64-column tile there would keep 12 of its 16 column lanes idle;
// instead the column lanes are regrouped as 4 column groups x 4 owner sub-tiles and every thread
// owns one row (RO_ = 1) of its sub-tile, so all 256 threads work on the 64 owners x 16 columns.
template <int MODEL, int P, bool OWNER_POS, int RO, bool MF, bool NARROW = false>
__device__ __forceinline__ void bwd_tile_body(const TileArgs &a, int lid, float *smem, int col_base = 0)
{
    static_assert(!(NARROW && MF), "the matrix-core loop has no narrow form");
    constexpr int RO_ = NARROW ? 1 : RO;           // owners per thread
    constexpr int TO = NARROW ? 64 : 16 * RO;      // owners per tile
    constexpr bool kRot = MODEL == KGE_ROTATE, kTH = MODEL == KGE_TRANSH;
    constexpr bool kDot = MODEL == KGE_DISTMULT || MODEL == KGE_COMPLEX || MODEL == KGE_TRANSF ||
                          MODEL == KGE_RESCAL;  // score = query . t' (+ const)
    constexpr bool kMf = kDot && MF;  // the sum over loopers on the matrix cores (else on the vector ALUs)
    constexpr bool kL2 = (MODEL == KGE_TRANSE || kTH) && P == 2;
    // L1 translation models: owner and looper rows carry the factor 2^100, so the sign of a residual
    // element is a single clamp (sgn_of_scaled, tile_common.hpp); the coefficient that multiplies a
    // scaled row (TransH: e) carries 2^-100
    constexpr bool kSc = (MODEL == KGE_TRANSE || kTH) && P == 1;
    constexpr int NPL = (kRot || (kTH && !OWNER_POS)) ? 2 : 1;  // looper planes in LDS
    constexpr int NPO = (kRot || (kTH && OWNER_POS)) ? 2 : 1;   // owner planes in registers
    constexpr int NC = kTH ? 3 : 1;                             // coefficient planes: g~, c, e
    constexpr int NOUT = (kRot || (kTH && OWNER_POS)) ? 2 : 1;
    constexpr int PG = TO + 4;
    constexpr int kKL = looper_rows<MODEL, RO>();  // (narrow tiles share the 64-owner launch and its step)
    constexpr int SL = kKL / 16;                        // looper float4 per thread per plane
    constexpr int CPT = (TO * kKL / 4 + 255) / 256;     // coefficient float4 per thread per plane
    static_assert(!NARROW || RO == 4, "narrow tiles share the 64-owner LDS layout");

    float(*sL)[kKL][kLP] = reinterpret_cast<float(*)[kKL][kLP]>(smem);
    float(*sG)[kKL][PG] = reinterpret_cast<float(*)[kKL][PG]>(smem + NPL * kKL * kLP);

    const int tid = threadIdx.x, tx = tid & 15, ty = tid >> 4;
    const int d = a.d, half = d >> 1;
    const int klen = pair_len<MODEL>(d);
    const int n_own = OWNER_POS ? a.C : a.N, n_loop = OWNER_POS ? a.N : a.C;
    int c, tile_y, tile_x;
    // wide tiles cover the columns [0, tiles_x * 64); a narrow tile the 16 columns from col_base on
    constexpr bool kHasNarrow = RO == 4 && !MF;  // launches of this shape hand a short remainder to narrow tiles
    // ComplEx on the matrix cores (128-bit rows): a column tile is 32 real columns and the matching 32
    // imaginary ones, [32 x, 32 x + 32) and half + [32 x, 32 x + 32), so that one workgroup holds both parts of
    // every complex element it owns (the positive chain in the epilogue needs them together, and a staging
    // step asks for half as many distinct row pieces of h and r)
    const bool pair = MODEL == KGE_COMPLEX && MF && !NARROW && a.vec != 0;
    const int wide_tiles_x = pair ? (half + 31) / 32
                                  : ((kHasNarrow && narrow_cols(klen)) ? klen / kTI : (klen + kTI - 1) / kTI);
    if (!xcd_tile(lid, NARROW ? 1 : wide_tiles_x, (n_own + TO - 1) / TO, a.n_chunks, c, tile_y, tile_x)) return;
    // local column lc (a multiple of 4 in 0..63) of the tile -> column of the row; and `lim` where the tile has
    // that column, else 0 (a paired tile's last columns may lie beyond the half row)
    auto gcol = [&](int lc) { return pair ? (lc < 32 ? tile_x * 32 + lc : half + tile_x * 32 + (lc - 32)) : (NARROW ? col_base : tile_x * kTI) + lc; };
    auto climit = [&](int lc, int lim) { return (pair && tile_x * 32 + (lc & 31) >= half) ? 0 : lim; };
    const int scol = gcol(tx * 4);                                           // columns this thread stages
    const int ctx = NARROW ? (tx & 3) : tx;                                  // column lane it computes
    const int col = gcol(ctx * 4);                                           // columns it owns
    const int ot0 = tile_y * TO;
    auto orow = [&](int o) { return NARROW ? (tx >> 2) * 16 + ty : ty * RO_ + o; };  // owner row inside the tile
    const bool vec = a.vec != 0;

    // ---- owners: registers -----------------------------------------------------------
    float4 own[NPO][RO_];
    float alo[RO_];
    auto load_owners = [&](auto vtag) {
    constexpr bool VEC = decltype(vtag)::value;
#pragma unroll
    for (int o = 0; o < RO_; ++o) {
        const int ol = ot0 + orow(o);
        const int lim = climit(ctx * 4, ol < n_own ? klen : 0);
        const int oc = ol < n_own ? ol : n_own - 1;
        alo[o] = 0.0f;
        if constexpr (OWNER_POS) {
            const int64_t b = (int64_t)c * a.C + oc;
            const int64_t rid = a.r[b];
            if constexpr (kTH) alo[o] = a.side_pos[b];
            float4 q0 = zero4(), q1 = zero4();
            if constexpr (!kDot)
                load_query<MODEL, VEC>(a.ent + a.h[b] * (int64_t)d, a.rel + rid * (int64_t)a.rel_dim,
                                  kTH ? a.aux + rid * (int64_t)d : nullptr, alo[o], col, lim, half, q0,
                                  q1, kRot ? a.query + b * (int64_t)d : nullptr, a.rsign);
            own[0][o] = q0;
            if constexpr (NPO == 2) own[1][o] = q1;
        } else {
            const float *pt = a.ent + a.neg[(int64_t)c * a.N + oc] * (int64_t)d;
            own[0][o] = kDot ? zero4() : ld4<VEC>(pt, col, lim);
            if constexpr (NPO == 2) own[1][o] = ld4<VEC>(pt + half, col, lim);
        }
        if constexpr (kSc) {
#pragma unroll
            for (int q = 0; q < NPO; ++q) own[q][o] = scale4(own[q][o], kSgnScale);
        }
    }
    };
    if (vec) load_owners(std::true_type{});
    else load_owners(std::false_type{});

    float4 acc[NOUT][RO_];
#pragma unroll
    for (int q = 0; q < NOUT; ++q)
#pragma unroll
        for (int o = 0; o < RO_; ++o) acc[q][o] = zero4();

    // DistMult / ComplEx: the sum over loopers is a plain matrix product, coefficients (owners x
    // loopers) times looper rows (loopers x columns), so it runs on the matrix cores
    // (v_mfma_f32_16x16x4_f32).  Lane l supplies A[i = l % 16][k = l / 16] and B[k][j = l % 16] and
    // receives D[i = 4 (l / 16) + v][j].  Inside 16 loopers the MFMA step s pairs lane group
    // g = l / 16 with looper 4 g + s; a lane's 128-bit read of four consecutive columns of that
    // looper's row feeds four MFMAs, so MFMA e owns the columns 4 j + e.  A wave owns 16 owners and
    // all 64 columns (64-owner tiles), or 16 owners and the columns 4 j + {0,1} / {2,3} (32-owner tiles).
    constexpr int OB = TO / 16, EW = OB;  // owner blocks; MFMAs (columns per lane) per wave
    static_assert(!kMf || OB == 4 || OB == 2, "MFMA tiling written for 32- and 64-owner tiles");
    const int mlane = tid & 63, mwave = tid >> 6, fj = mlane & 15, fg = mlane >> 4;
    const int ob = mwave % OB, e0 = (mwave / OB) * EW;
    v4f macc[EW];
#pragma unroll
    for (int e = 0; e < EW; ++e) macc[e] = v4f{0.0f, 0.0f, 0.0f, 0.0f};

    // ---- staging: a three-deep software pipeline --------------------------------------------
    // While step st is computed, the rows and coefficients of step st+1 are in flight and so are
    // the looper INDICES of step st+2 (h / r / neg ids, TransH w.h): the dependent chain
    // "index -> row address -> row" never stalls a step.  The prefetch registers hold raw loads
    // (load_query_raw); they are combined into query rows / scaled coefficients only when the
    // step is written to LDS, so nothing waits on them before the compute.  TransH keeps the
    // combine at load time: its register budget has no room for the raw operands.
    constexpr bool kDefer = !kTH;
    constexpr int NRAW = OWNER_POS ? NPL : (kDefer ? query_raw_count<MODEL>() : NPL);
    constexpr int NCR = kTH ? 3 : (kL2 ? 2 : 1);  // raw coefficient planes: dneg, (sneg | side_neg x 2)
    float4 rraw[SL][NRAW];
    float4 craw[NCR][CPT];
    int64_t li0[SL], li1[SL];  // looper ids: negative entity, or (kept entity, relation) of a positive
    float lal[SL];             // TransH: w . x of a looper positive

    auto load_idx = [&](int l0) {
#pragma unroll
        for (int s = 0; s < SL; ++s) {
            const int ll = l0 + ty + 16 * s;
            const int lc = ll < n_loop ? ll : n_loop - 1;
            if constexpr (OWNER_POS) {
                li0[s] = a.neg[(int64_t)c * a.N + lc];
            } else {
                const int64_t b = (int64_t)c * a.C + lc;
                li0[s] = a.h[b], li1[s] = a.r[b];
                if constexpr (kTH) lal[s] = a.side_pos[b];
            }
        }
    };

    auto load_rows_v = [&](auto vtag, auto ntag, int l0) {
        constexpr bool VEC = decltype(vtag)::value, VECN = decltype(ntag)::value;
        // looper rows: thread stages rows ty + 16*s, columns col..col+3
#pragma unroll
        for (int s = 0; s < SL; ++s) {
            const int ll = l0 + ty + 16 * s;
            const int lim = climit(tx * 4, ll < n_loop ? klen : 0);
            if constexpr (OWNER_POS) {
                const float *pt = a.ent + li0[s] * (int64_t)d;
                rraw[s][0] = ld4_raw<VEC>(pt, scol, lim);
                if constexpr (NPL == 2) rraw[s][1] = ld4_raw<VEC>(pt + half, scol, lim);
            } else {
                const int64_t b = (int64_t)c * a.C + (ll < n_loop ? ll : n_loop - 1);
                const float *ph = a.ent + li0[s] * (int64_t)d, *pr = a.rel + li1[s] * (int64_t)a.rel_dim;
                const float *pw = kTH ? a.aux + li1[s] * (int64_t)d : nullptr;
                const float *pq = (kRot || MODEL == KGE_RESCAL) ? a.query + b * (int64_t)d : nullptr;
                if constexpr (kDefer) {
                    load_query_raw<MODEL, VEC>(ph, pr, pw, pq, scol, lim, half, rraw[s]);
                } else {
                    load_query<MODEL, VEC>(ph, pr, pw, lal[s], scol, lim, half, rraw[s][0], rraw[s][NRAW - 1], pq, a.rsign);
                }
            }
        }
        // coefficients of the (TO owners x kKL loopers) block, read along k (contiguous)
#pragma unroll
        for (int s = 0; s < CPT; ++s) {
            const int f = tid + 256 * s;  // float4 index inside the block
            int bl, kl;                   // positive / negative of the first element
            bool inside;
            if constexpr (OWNER_POS) {    // rows = owners (positives), kKL / 4 float4 of loopers each
                const int orow = f / (kKL / 4);
                bl = ot0 + orow, kl = l0 + (f % (kKL / 4)) * 4;
                inside = orow < TO && bl < a.C;
            } else {                      // rows = loopers (positives), TO/4 float4 of owners each
                const int lrow = f / (TO / 4);
                bl = l0 + lrow, kl = ot0 + (f % (TO / 4)) * 4;
                inside = lrow < kKL && bl < a.C;
            }
            const int lim = inside ? a.N : 0;
            const int64_t off = ((int64_t)c * a.C + (inside ? bl : 0)) * a.N;
            craw[0][s] = ld4<VECN>(a.dneg + off, kl, lim);
            if constexpr (kL2 && !kTH) craw[1][s] = ld4<VECN>(a.sneg + off, kl, lim);
            if constexpr (kTH) {
                craw[1][s] = ld4<VECN>(a.side_neg + off, kl, lim);
                craw[2][s] = ld4<VECN>(a.side_neg + a.plane + off, kl, lim);
                if constexpr (kL2) {  // fold the norm in now (TransH does not defer)
                    const float4 sc = ld4<VECN>(a.sneg + off, kl, lim);
                    float4 &g = craw[0][s];
                    craw[2][s] = mul4(g, craw[2][s]);
                    g.x = sc.x > 0.0f ? g.x / sc.x : 0.0f;
                    g.y = sc.y > 0.0f ? g.y / sc.y : 0.0f;
                    g.z = sc.z > 0.0f ? g.z / sc.z : 0.0f;
                    g.w = sc.w > 0.0f ? g.w / sc.w : 0.0f;
                } else {
                    craw[2][s] = mul4(scale4(craw[0][s], kSgnUnscale), craw[2][s]);  // kSc: multiplies a scaled row
                }
            }
        }
    };

    auto load_rows = [&](int l0) {  // one uniform dispatch per step, no branch per load
        if (vec) {
            if (a.vecn) load_rows_v(std::true_type{}, std::true_type{}, l0);
            else load_rows_v(std::true_type{}, std::false_type{}, l0);
        } else {
            if (a.vecn) load_rows_v(std::false_type{}, std::true_type{}, l0);
            else load_rows_v(std::false_type{}, std::false_type{}, l0);
        }
    };

    auto store_step_v = [&](auto vtag, int l0) {
        constexpr bool VEC = decltype(vtag)::value;
#pragma unroll
        for (int s = 0; s < SL; ++s) {
            float4 q0, q1 = zero4();
            if constexpr (OWNER_POS || !kDefer) {
                q0 = rraw[s][0];
                if constexpr (NPL == 2) q1 = rraw[s][NRAW - 1];
            } else {
                const int ll = l0 + ty + 16 * s;
                combine_query<MODEL, VEC>(rraw[s], 0.0f, scol, climit(tx * 4, ll < n_loop ? klen : 0), half, a.rsign, q0, q1);
            }
            if constexpr (kSc) q0 = scale4(q0, kSgnScale), q1 = scale4(q1, kSgnScale);
            *reinterpret_cast<float4 *>(&sL[0][ty + 16 * s][tx * 4]) = q0;
            if constexpr (NPL == 2) *reinterpret_cast<float4 *>(&sL[1][ty + 16 * s][tx * 4]) = q1;
        }
#pragma unroll
        for (int s = 0; s < CPT; ++s) {
            const int f = tid + 256 * s;
            float4 cv[NC];
            cv[0] = craw[0][s];
            if constexpr (kL2 && !kTH) {
                const float4 sc = craw[1][s];
                cv[0].x = sc.x > 0.0f ? cv[0].x / sc.x : 0.0f;
                cv[0].y = sc.y > 0.0f ? cv[0].y / sc.y : 0.0f;
                cv[0].z = sc.z > 0.0f ? cv[0].z / sc.z : 0.0f;
                cv[0].w = sc.w > 0.0f ? cv[0].w / sc.w : 0.0f;
            }
            if constexpr (kTH) cv[1] = craw[1][s], cv[2] = craw[2][s];
#pragma unroll
            for (int pl = 0; pl < NC; ++pl) {
                const float4 v = cv[pl];
                if constexpr (OWNER_POS) {
                    const int orow = f / (kKL / 4), l = (f % (kKL / 4)) * 4;
                    if (orow < TO) {
                        sG[pl][l + 0][orow] = v.x;
                        sG[pl][l + 1][orow] = v.y;
                        sG[pl][l + 2][orow] = v.z;
                        sG[pl][l + 3][orow] = v.w;
                    }
                } else {
                    const int lrow = f / (TO / 4), o4 = (f % (TO / 4)) * 4;
                    if (lrow < kKL) *reinterpret_cast<float4 *>(&sG[pl][lrow][o4]) = v;
                }
            }
        }
    };
    auto store_step = [&](int l0) {
        if (vec) store_step_v(std::true_type{}, l0);
        else store_step_v(std::false_type{}, l0);
    };

    const int nstep = (n_loop + kKL - 1) / kKL;
    load_idx(0);
    load_rows(0);
    load_idx(kKL);  // clamped inside: harmless past the end
#pragma unroll 1
    for (int st = 0; st < nstep; ++st) {
        store_step(st * kKL);
        __syncthreads();
        if (st + 1 < nstep) {
            load_rows((st + 1) * kKL);
            load_idx((st + 2) * kKL);
        }
        // two-level sum: the kKL loopers of a step go into a fresh accumulator that is folded
        // into the running one per step, so rounding grows with sqrt(steps) of the large partial
        // sums instead of sqrt(loopers)
        if constexpr (kMf) {
#pragma unroll
            for (int q = 0; q < kKL / 16; ++q)
#pragma unroll
                for (int ms = 0; ms < 4; ++ms) {
                    const int l = 16 * q + 4 * fg + ms;
                    const float av = sG[0][l][ob * 16 + fj];
                    float bv[EW];
                    if constexpr (EW == 4) {
                        const float4 b4 = *reinterpret_cast<const float4 *>(&sL[0][l][4 * fj]);
                        bv[0] = b4.x, bv[1] = b4.y, bv[2] = b4.z, bv[3] = b4.w;
                    } else {
                        const float2 b2 = *reinterpret_cast<const float2 *>(&sL[0][l][4 * fj + e0]);
                        bv[0] = b2.x, bv[1] = b2.y;
                    }
#pragma unroll
                    for (int e = 0; e < EW; ++e)
                        macc[e] = __builtin_amdgcn_mfma_f32_16x16x4f32(av, bv[e], macc[e], 0, 0, 0);
                }
        }
        float4 sacc[NOUT][RO_];
#pragma unroll
        for (int q = 0; q < NOUT; ++q)
#pragma unroll
            for (int o = 0; o < RO_; ++o) sacc[q][o] = zero4();
#pragma unroll 4
        for (int l = 0; l < (kMf ? 0 : kKL); ++l) {
            float4 lv[NPL];
#pragma unroll
            for (int pl = 0; pl < NPL; ++pl) lv[pl] = *reinterpret_cast<const float4 *>(&sL[pl][l][ctx * 4]);
#pragma unroll
            for (int o = 0; o < RO_; ++o) {
                const float g = sG[0][l][orow(o)];
                const float *lvp = reinterpret_cast<const float *>(&lv[0]);
                const float *lv1p = reinterpret_cast<const float *>(&lv[NPL - 1]);
                const float *o0p = reinterpret_cast<const float *>(&own[0][o]);
                const float *o1p = reinterpret_cast<const float *>(&own[NPO - 1][o]);
                float *a0p = reinterpret_cast<float *>(&sacc[0][o]);
                float *a1p = reinterpret_cast<float *>(&sacc[NOUT - 1][o]);
                if constexpr (kDot) {
#pragma unroll
                    for (int e = 0; e < 4; ++e) a0p[e] = fmaf(g, lvp[e], a0p[e]);
                } else if constexpr (MODEL == KGE_TRANSE) {
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        const float u = OWNER_POS ? o0p[e] - lvp[e] : lvp[e] - o0p[e];  // a - t' (P == 1: times 2^100)
                        const float ph = P == 1 ? sgn_of_scaled(u) : u;
                        a0p[e] = OWNER_POS ? fmaf(g, ph, a0p[e]) : fmaf(-g, ph, a0p[e]);
                    }
                } else if constexpr (kRot) {
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        const float ur = OWNER_POS ? o0p[e] - lvp[e] : lvp[e] - o0p[e];
                        const float ui = OWNER_POS ? o1p[e] - lv1p[e] : lv1p[e] - o1p[e];
                        // u == 0 contributes k * 0 = 0 whatever k is, so |u|^2 only has to stay away from zero:
                        // the 1e-37 rides in the multiply-add that forms it (far below one ulp of any |u|^2
                        // that is not itself denormal) instead of a compare-and-select or a max
                        const float m2 = fmaf(ur, ur, fmaf(ui, ui, 1e-37f));
                        const float rs = __builtin_amdgcn_rsqf(m2);
                        const float k = OWNER_POS ? -g * rs : g * rs;  // d/da = -g u/|u| ; d/dt' = +g u/|u|
                        a0p[e] = fmaf(k, ur, a0p[e]);
                        a1p[e] = fmaf(k, ui, a1p[e]);
                    }
                } else if constexpr (kTH) {
                    const float cc = sG[1][l][orow(o)], ee = sG[2][l][orow(o)];
                    if constexpr (OWNER_POS) {
                        // q = g phi(u) goes into a0 and, times -w.(h - t'_k), into a1: with the two
                        // coefficients formed once per pair, phi(u) feeds two multiply-adds directly
                        const float gk = -(alo[o] - cc) * g;
#pragma unroll
                        for (int e = 0; e < 4; ++e) {
                            const float u = fmaf(cc, o1p[e], o0p[e] - lvp[e]);
                            const float ph = P == 1 ? sgn_of_scaled(u) : u;
                            a0p[e] = fmaf(g, ph, a0p[e]);
                            a1p[e] = fmaf(ee, lvp[e], fmaf(gk, ph, a1p[e]));
                        }
                    } else {
#pragma unroll
                        for (int e = 0; e < 4; ++e) {
                            const float u = fmaf(cc, lv1p[e], lvp[e] - o0p[e]);
                            const float ph = P == 1 ? sgn_of_scaled(u) : u;
                            a0p[e] = fmaf(ee, lv1p[e], fmaf(-g, ph, a0p[e]));
                        }
                    }
                }
            }
        }
#pragma unroll
        for (int q = 0; q < NOUT; ++q)
#pragma unroll
            for (int o = 0; o < RO_; ++o) acc[q][o] = add4(acc[q][o], sacc[q][o]);
        __syncthreads();
    }

    if constexpr (kMf) {
        if constexpr (OWNER_POS && EW == 4 && (MODEL == KGE_DISTMULT || MODEL == KGE_COMPLEX)) {
            if (a.chain) {  // uniform: the positive chain right here, from the sums in the accumulators
                const int lc = 4 * fj;
                const int c0 = gcol(lc);
                const bool colok = climit(lc, klen) != 0 && c0 + 4 <= d;
                const int cc = colok ? c0 : 0;  // clamped: unconditional loads
                int64_t idk[4], ido[4], idr[4];
                float gp[4];
                bool rowok[4];
#pragma unroll
                for (int v = 0; v < 4; ++v) {
                    const int ol = ot0 + ob * 16 + 4 * fg + v;
                    rowok[v] = ol < n_own;
                    const int64_t b = (int64_t)c * a.C + (rowok[v] ? ol : n_own - 1);
                    idk[v] = a.h[b], ido[v] = a.other[b], idr[v] = a.r[b];
                    gp[v] = a.dpos ? a.dpos[b] : 0.0f;
                }
                if constexpr (MODEL == KGE_DISTMULT) {
                    float4 xk[4], xo[4], xr[4];
#pragma unroll
                    for (int v = 0; v < 4; ++v) {
                        xk[v] = *reinterpret_cast<const float4 *>(a.ent + idk[v] * (int64_t)d + cc);
                        xo[v] = *reinterpret_cast<const float4 *>(a.ent + ido[v] * (int64_t)d + cc);
                        xr[v] = *reinterpret_cast<const float4 *>(a.rel + idr[v] * (int64_t)a.rel_dim + cc);
                    }
#pragma unroll
                    for (int v = 0; v < 4; ++v) {
                        const float k4[4] = {xk[v].x, xk[v].y, xk[v].z, xk[v].w}, o4[4] = {xo[v].x, xo[v].y, xo[v].z, xo[v].w};
                        const float r4[4] = {xr[v].x, xr[v].y, xr[v].z, xr[v].w};
                        float dk[4], dr[4], dother[4];
#pragma unroll
                        for (int e = 0; e < 4; ++e) distmult_chain(gp[v], k4[e], o4[e], r4[e], macc[e][v], dk[e], dr[e], dother[e]);
                        if (rowok[v] && colok) {
                            const int64_t b = (int64_t)c * a.C + ot0 + ob * 16 + 4 * fg + v;
                            *reinterpret_cast<float4 *>(a.occ_k + b * (int64_t)d + c0) = make_float4(dk[0], dk[1], dk[2], dk[3]);
                            *reinterpret_cast<float4 *>(a.occ_r + b * (int64_t)a.rel_dim + c0) = make_float4(dr[0], dr[1], dr[2], dr[3]);
                            *reinterpret_cast<float4 *>(a.occ_o + b * (int64_t)d + c0) = make_float4(dother[0], dother[1], dother[2], dother[3]);
                        }
                    }
                } else {
                    // lanes fj < 8 hold the real parts of complex elements idx .. idx + 3, lanes fj + 8 the imaginary
                    // parts of the same elements: each takes the other part from its partner and writes its own side
                    const bool is_re = fj < 8;
                    const int idx = tile_x * 32 + 4 * (fj & 7);
                    const int ci = colok ? idx : 0;
#pragma unroll
                    for (int v = 0; v < 4; ++v) {
                        float Gm[4], Gp[4];
#pragma unroll
                        for (int e = 0; e < 4; ++e) Gm[e] = macc[e][v], Gp[e] = __shfl_xor(macc[e][v], 8, kWave);
                        const float *pk = a.ent + idk[v] * (int64_t)d + ci, *po = a.ent + ido[v] * (int64_t)d + ci;
                        const float *pr = a.rel + idr[v] * (int64_t)a.rel_dim + ci;
                        const float4 kr4 = *reinterpret_cast<const float4 *>(pk), ki4 = *reinterpret_cast<const float4 *>(pk + half);
                        const float4 or4 = *reinterpret_cast<const float4 *>(po), oi4 = *reinterpret_cast<const float4 *>(po + half);
                        const float4 qr4 = *reinterpret_cast<const float4 *>(pr), qi4 = *reinterpret_cast<const float4 *>(pr + half);
                        const float kr[4] = {kr4.x, kr4.y, kr4.z, kr4.w}, ki[4] = {ki4.x, ki4.y, ki4.z, ki4.w};
                        const float orr[4] = {or4.x, or4.y, or4.z, or4.w}, oi[4] = {oi4.x, oi4.y, oi4.z, oi4.w};
                        const float qr[4] = {qr4.x, qr4.y, qr4.z, qr4.w}, qi[4] = {qi4.x, qi4.y, qi4.z, qi4.w};
                        float dk[4], dr[4], dother[4];
#pragma unroll
                        for (int e = 0; e < 4; ++e) {
                            const float Gr = is_re ? Gm[e] : Gp[e], Gi = is_re ? Gp[e] : Gm[e];
                            float dkr, dki, drr, dri, dor, doi;
                            if (a.rsign < 0.0f) complex_chain<true>(gp[v], kr[e], ki[e], orr[e], oi[e], qr[e], qi[e], Gr, Gi, dkr, dki, drr, dri, dor, doi);
                            else complex_chain<false>(gp[v], kr[e], ki[e], orr[e], oi[e], qr[e], qi[e], Gr, Gi, dkr, dki, drr, dri, dor, doi);
                            dk[e] = is_re ? dkr : dki, dr[e] = is_re ? drr : dri, dother[e] = is_re ? dor : doi;
                        }
                        if (rowok[v] && colok) {
                            const int64_t b = (int64_t)c * a.C + ot0 + ob * 16 + 4 * fg + v;
                            *reinterpret_cast<float4 *>(a.occ_k + b * (int64_t)d + c0) = make_float4(dk[0], dk[1], dk[2], dk[3]);
                            *reinterpret_cast<float4 *>(a.occ_r + b * (int64_t)a.rel_dim + c0) = make_float4(dr[0], dr[1], dr[2], dr[3]);
                            *reinterpret_cast<float4 *>(a.occ_o + b * (int64_t)d + c0) = make_float4(dother[0], dother[1], dother[2], dother[3]);
                        }
                    }
                }
                return;
            }
        }
#pragma unroll
        for (int v = 0; v < 4; ++v) {
            const int ol = ot0 + ob * 16 + 4 * fg + v;
            if (ol >= n_own) continue;
            const int64_t row = OWNER_POS ? (int64_t)c * a.C + ol : (int64_t)c * a.N + ol;
            float *dst = a.out0 + row * (int64_t)d;
            const int c0 = gcol(4 * fj + e0);
            if (pair && climit(4 * fj + e0, klen) == 0) continue;
            if (vec && c0 + EW <= klen) {  // rows 16-byte aligned and d % 4 == 0: whole group inside
                if constexpr (EW == 4)
                    *reinterpret_cast<float4 *>(dst + c0) = make_float4(macc[0][v], macc[1][v], macc[2][v], macc[3][v]);
                else
                    *reinterpret_cast<float2 *>(dst + c0) = make_float2(macc[0][v], macc[1][v]);
            } else {
#pragma unroll
                for (int e = 0; e < EW; ++e)
                    if (c0 + e < klen) dst[c0 + e] = macc[e][v];
            }
        }
        return;
    }
#pragma unroll
    for (int o = 0; o < RO_; ++o) {
        const int ol = ot0 + orow(o);
        if (ol >= n_own) continue;
        const int64_t row = OWNER_POS ? (int64_t)c * a.C + ol : (int64_t)c * a.N + ol;
        float *dst = a.out0 + row * (int64_t)d;
        st4(dst, col, klen, vec, acc[0][o]);
        if constexpr (kRot) st4(dst + half, col, klen, vec, acc[1][o]);
        if constexpr (kTH && OWNER_POS) st4(a.out1 + row * (int64_t)d, col, klen, vec, acc[1][o]);
    }
}

// Both orientations in ONE launch: the first `grid_head` workgroups own positives (outputs
// g0 / g1), the rest own negatives (output occ_neg).  The two halves are independent, and
// together they fill the GPU better than either alone when the batch is small.
// Workgroup ranges of a launch, in order: the inspector's riders, wide tiles owning positives,
// wide tiles owning negatives, then (64-owner vector-ALU launches only, when the row width leaves
// a remainder of at most 16 columns) narrow tiles owning positives and narrow tiles owning negatives.
struct TileGrid {
    int head, neg, narrow_head, narrow_neg;
};

template <int MODEL, int P, int RO, bool MF>
__global__ __launch_bounds__(256, KGE_TILE_OCC) void bwd_tile_kernel(TileArgs a, float *g0, float *g1, float *occ_neg,
                                                                     TileGrid grid, FusedInsp fi)
{
    extern __shared__ __align__(16) char dyn_smem[];  // tile_lds_bytes<MODEL, RO>() or the inspector's need
    if (fused_insp_block(fi, reinterpret_cast<uint32_t *>(dyn_smem))) return;
    float *smem = reinterpret_cast<float *>(dyn_smem);
    int lid = (int)blockIdx.x - fi.blocks;
    if (lid < grid.head) {
        a.out0 = g0, a.out1 = g1;
        bwd_tile_body<MODEL, P, true, RO, MF>(a, lid, smem);
        return;
    }
    lid -= grid.head;
    if (lid < grid.neg) {
        a.out0 = occ_neg, a.out1 = nullptr;
        bwd_tile_body<MODEL, P, false, RO, MF>(a, lid, smem);
        return;
    }
    if constexpr (RO == 4 && !MF) {
        lid -= grid.neg;
        const int klen = pair_len<MODEL>(a.d);
        const int col_base = (klen / kTI) * kTI;
        if (lid < grid.narrow_head) {
            a.out0 = g0, a.out1 = g1;
            bwd_tile_body<MODEL, P, true, RO, MF, true>(a, lid, smem, col_base);
        } else {
            a.out0 = occ_neg, a.out1 = nullptr;
            bwd_tile_body<MODEL, P, false, RO, MF, true>(a, lid - grid.narrow_head, smem, col_base);
        }
    }
}

template <int MODEL, int RO>
static size_t tile_lds_bytes(const FusedInsp &fi)
{
    constexpr int kFloats = TileShape<MODEL, true, RO>::kLdsFloats > TileShape<MODEL, false, RO>::kLdsFloats
                                ? TileShape<MODEL, true, RO>::kLdsFloats
                                : TileShape<MODEL, false, RO>::kLdsFloats;
    const size_t own = sizeof(float) * kFloats;
    return fi.blocks > 0 && (size_t)fi.lds_bytes > own ? (size_t)fi.lds_bytes : own;
}

template <int MODEL, int P>
static int launch_tiles(TileArgs a, float *g0, float *g1, float *occ_neg, int64_t n_chunks, bool dot_valu,
                        const FusedInsp &fi, hipStream_t st)
{
    const int klen = MODEL == KGE_ROTATE ? a.d / 2 : a.d;
    const int64_t gx = ceil_div(klen, kTI);
    const bool narrow = narrow_cols(klen) > 0;       // the last 1..16 columns go to narrow tiles (64-owner VALU launches)
    const int64_t gxw = narrow ? klen / kTI : gx;    // wide column tiles of such a launch
    const int64_t big = gx * (ceil_div(a.C, 64) + ceil_div(a.N, 64)) * n_chunks;
    // the size rule follows launch_neg_mp (see there)
    constexpr bool kDotModel = MODEL == KGE_DISTMULT || MODEL == KGE_COMPLEX || MODEL == KGE_TRANSF || MODEL == KGE_RESCAL;
    if constexpr (kDotModel) {
        // matrix-core inner loop (KGE_PAIR_SUMS_VALU keeps the vector-ALU loop): a wave gets all 64
        // columns of its 16 owners with 64-owner tiles, which win at every size
        if (!dot_valu) {
            // (ComplEx with 128-bit rows: column tiles pair 32 real with the matching 32 imaginary columns)
            const int64_t gxm = (MODEL == KGE_COMPLEX && a.vec) ? ceil_div(a.d / 2, 32) : gx;
            const unsigned gh = xcd_grid(gxm, ceil_div(a.C, 64), n_chunks), gn = xcd_grid(gxm, ceil_div(a.N, 64), n_chunks);
            const size_t lds = tile_lds_bytes<MODEL, 4>(fi);
            hipLaunchKernelGGL((bwd_tile_kernel<MODEL, P, 4, true>), dim3(gh + gn + fi.blocks), dim3(256), lds, st, a,
                               g0, g1, occ_neg, TileGrid{(int)gh, (int)gn, 0, 0}, fi);
            KGE_CHECK_LAUNCH();
            return KGE_OK;
        }
    }
    if (big >= 1024) {
        const unsigned gh = xcd_grid(gxw, ceil_div(a.C, 64), n_chunks), gn = xcd_grid(gxw, ceil_div(a.N, 64), n_chunks);
        const unsigned nh = narrow ? xcd_grid(1, ceil_div(a.C, 64), n_chunks) : 0;
        const unsigned nn = narrow ? xcd_grid(1, ceil_div(a.N, 64), n_chunks) : 0;
        const size_t lds = tile_lds_bytes<MODEL, 4>(fi);
        hipLaunchKernelGGL((bwd_tile_kernel<MODEL, P, 4, false>), dim3(gh + gn + nh + nn + fi.blocks), dim3(256), lds, st,
                           a, g0, g1, occ_neg, TileGrid{(int)gh, (int)gn, (int)nh, (int)nn}, fi);
    } else if (big >= 512) {
        const unsigned gh = xcd_grid(gx, ceil_div(a.C, 32), n_chunks), gn = xcd_grid(gx, ceil_div(a.N, 32), n_chunks);
        const size_t lds = tile_lds_bytes<MODEL, 2>(fi);
        hipLaunchKernelGGL((bwd_tile_kernel<MODEL, P, 2, false>), dim3(gh + gn + fi.blocks), dim3(256), lds, st, a, g0, g1,
                           occ_neg, TileGrid{(int)gh, (int)gn, 0, 0}, fi);
    } else {
        // a batch this small leaves one or two 32-owner workgroups per CU: 16-owner tiles double the
        // waves that hide each other's latency
        const unsigned gh = xcd_grid(gx, ceil_div(a.C, 16), n_chunks), gn = xcd_grid(gx, ceil_div(a.N, 16), n_chunks);
        const size_t lds = tile_lds_bytes<MODEL, 1>(fi);
        hipLaunchKernelGGL((bwd_tile_kernel<MODEL, P, 1, false>), dim3(gh + gn + fi.blocks), dim3(256), lds, st, a, g0, g1,
                           occ_neg, TileGrid{(int)gh, (int)gn, 0, 0}, fi);
    }
    KGE_CHECK_LAUNCH();
    return KGE_OK;
}

// ---------------------------------------------------------------------------------------
// 3: one wave per positive triple
// ---------------------------------------------------------------------------------------
struct PosBwdArgs {
    const float *ent, *rel, *aux;
    const int64_t *h, *r, *t;
    const float *dpos, *spos, *side_pos;
    const float *g0, *g1;  // [B, d] accumulations over the negatives (may be null)
    const float *dneg;     // TransF with negatives: [B, N] upstream gradient (its row sums scale the constant's gradient)
    int64_t N;
    float *occ_h, *occ_t;  // [B, d] each
    float *occ_r;          // [B, rel_dim]
    float *occ_w;          // [B, d] TransH
    int64_t B;
    int d, rel_dim;
};

template <int V>
__device__ __forceinline__ Vec<V> ldz(const float *p, int j)
{
    if (p) return Vec<V>::load(p + j);
    Vec<V> z;
#pragma unroll
    for (int e = 0; e < V; ++e) z.v[e] = 0.0f;
    return z;
}

// G (g0) is the gradient with respect to the query row a_b accumulated over the chunk's negatives.
// With negatives that replace the tail the query is built from (h, r); with HEAD it is built from
// (x, rho) = (t, -r) [TransE, TransH], (t, conj r) [ComplEx], (t, -theta) [RotatE], (t, r) [DistMult],
// so G chains into the t and r rows instead and the positive triple's own term is kept apart.
template <int MODEL, int P, int V, bool HEAD>
__global__ __launch_bounds__(256) void bwd_pos_kernel(PosBwdArgs a, FusedInsp fi)
{
    extern __shared__ __align__(16) char dyn_smem[];  // inspector workgroups only
    if (fused_insp_block(fi, reinterpret_cast<uint32_t *>(dyn_smem))) return;
    const int lane = threadIdx.x & (kWave - 1);
    const int64_t b = (int64_t)((int)blockIdx.x - fi.blocks) * 4 + (threadIdx.x >> 6);
    if (b >= a.B) return;  // whole waves leave together; no block-level sync below
    const int d = a.d, half = d >> 1;
    const int64_t rid = a.r[b];
    const float *eh = a.ent + a.h[b] * (int64_t)d, *et = a.ent + a.t[b] * (int64_t)d;
    const float *rr = a.rel ? a.rel + rid * (int64_t)a.rel_dim : nullptr;
    const float *g0 = a.g0 ? a.g0 + b * (int64_t)d : nullptr;
    const float *g1 = a.g1 ? a.g1 + b * (int64_t)d : nullptr;
    float *oh = a.occ_h + b * (int64_t)d, *ot = a.occ_t + b * (int64_t)d;
    float *orr = a.occ_r ? a.occ_r + b * (int64_t)a.rel_dim : nullptr;
    const float g = a.dpos ? a.dpos[b] : 0.0f;
    float gs = g;  // g / ||u|| for the L2 models
    if constexpr ((MODEL == KGE_TRANSE || MODEL == KGE_TRANSH) && P == 2) {
        const float s = a.spos[b];
        gs = s > 0.0f ? g / s : 0.0f;
    }

    if constexpr (MODEL == KGE_TRANSE) {
        for (int j = lane * V; j < d; j += kWave * V) {
            const Vec<V> vh = Vec<V>::load(eh + j), vt = Vec<V>::load(et + j), vr = Vec<V>::load(rr + j);
            const Vec<V> G = ldz<V>(g0, j);
            Vec<V> dh, dt;
#pragma unroll
            for (int e = 0; e < V; ++e) {
                const float u = (vh.v[e] - vt.v[e]) + vr.v[e];
                const float q = gs * (P == 1 ? sgn(u) : u);
                dh.v[e] = HEAD ? q : q + G.v[e];
                dt.v[e] = HEAD ? G.v[e] - q : -q;
            }
            if constexpr (HEAD) {
                Vec<V> dr;
#pragma unroll
                for (int e = 0; e < V; ++e) dr.v[e] = dh.v[e] - G.v[e];
                dr.store(orr + j);
            } else {
                dh.store(orr + j);
            }
            dh.store(oh + j), dt.store(ot + j);
        }
    } else if constexpr (MODEL == KGE_DISTMULT) {
        for (int j = lane * V; j < d; j += kWave * V) {
            const Vec<V> vh = Vec<V>::load(eh + j), vt = Vec<V>::load(et + j), vr = Vec<V>::load(rr + j);
            const Vec<V> G = ldz<V>(g0, j);
            Vec<V> dh, dr, dt;
#pragma unroll
            for (int e = 0; e < V; ++e) {
                if constexpr (HEAD) distmult_chain(g, vt.v[e], vh.v[e], vr.v[e], G.v[e], dt.v[e], dr.v[e], dh.v[e]);  // a = t * r
                else distmult_chain(g, vh.v[e], vt.v[e], vr.v[e], G.v[e], dh.v[e], dr.v[e], dt.v[e]);
            }
            dh.store(oh + j), dr.store(orr + j), dt.store(ot + j);
        }
    } else if constexpr (MODEL == KGE_TRANSF) {
        // pair score (2x + rs r).n - rs r.x with x the kept side (h; t with HEAD, rs = -1): G = sum_k dneg n_k
        // chains with 2 into x and rs into r; the constant's gradient is -rs S r (to x) and -rs S x (to r),
        // S = sum_k dneg[b][k]
        float S = 0.0f;
        if (a.dneg && g0) {  // uniform
            for (int64_t k = lane; k < a.N; k += kWave) S += a.dneg[b * a.N + k];
            S = wave_sum(S);
        }
        for (int j = lane * V; j < d; j += kWave * V) {
            const Vec<V> vh = Vec<V>::load(eh + j), vt = Vec<V>::load(et + j), vr = Vec<V>::load(rr + j);
            const Vec<V> G = ldz<V>(g0, j);
            Vec<V> dh, dr, dt;
#pragma unroll
            for (int e = 0; e < V; ++e) {
                dh.v[e] = g * (2.0f * vt.v[e] - vr.v[e]);
                dt.v[e] = g * (2.0f * vh.v[e] + vr.v[e]);
                dr.v[e] = g * (vt.v[e] - vh.v[e]);
                if constexpr (HEAD) {
                    dt.v[e] += fmaf(S, vr.v[e], 2.0f * G.v[e]);
                    dr.v[e] += fmaf(S, vt.v[e], -G.v[e]);
                } else {
                    dh.v[e] += fmaf(-S, vr.v[e], 2.0f * G.v[e]);
                    dr.v[e] += fmaf(-S, vh.v[e], G.v[e]);
                }
            }
            dh.store(oh + j), dr.store(orr + j), dt.store(ot + j);
        }
    } else if constexpr (MODEL == KGE_COMPLEX) {
        for (int j = lane * V; j < half; j += kWave * V) {
            const Vec<V> hr = Vec<V>::load(eh + j), hi = Vec<V>::load(eh + half + j);
            const Vec<V> tr = Vec<V>::load(et + j), ti = Vec<V>::load(et + half + j);
            const Vec<V> qr = Vec<V>::load(rr + j), qi = Vec<V>::load(rr + half + j);
            const Vec<V> Gr = ldz<V>(g0, j), Gi = ldz<V>(g0, half + j);
            Vec<V> dhr, dhi, drr, dri, dtr, dti;
#pragma unroll
            for (int e = 0; e < V; ++e) {
                if constexpr (HEAD)  // s = Re<n, r, conj t> = n . (conj(r) o t): a = conj(r) o t, Q = g h + G
                    complex_chain<true>(g, tr.v[e], ti.v[e], hr.v[e], hi.v[e], qr.v[e], qi.v[e], Gr.v[e], Gi.v[e], dtr.v[e], dti.v[e],
                                        drr.v[e], dri.v[e], dhr.v[e], dhi.v[e]);
                else
                    complex_chain<false>(g, hr.v[e], hi.v[e], tr.v[e], ti.v[e], qr.v[e], qi.v[e], Gr.v[e], Gi.v[e], dhr.v[e], dhi.v[e],
                                         drr.v[e], dri.v[e], dtr.v[e], dti.v[e]);
            }
            dhr.store(oh + j), dhi.store(oh + half + j);
            drr.store(orr + j), dri.store(orr + half + j);
            dtr.store(ot + j), dti.store(ot + half + j);
        }
    } else if constexpr (MODEL == KGE_ROTATE) {
        for (int j = lane * V; j < half; j += kWave * V) {
            const Vec<V> hr = Vec<V>::load(eh + j), hi = Vec<V>::load(eh + half + j);
            const Vec<V> tr = Vec<V>::load(et + j), ti = Vec<V>::load(et + half + j);
            const Vec<V> th = Vec<V>::load(rr + j);
            const Vec<V> Gr = ldz<V>(g0, j), Gi = ldz<V>(g0, half + j);
            Vec<V> dhr, dhi, dth, dtr, dti;
#pragma unroll
            for (int e = 0; e < V; ++e) {
                float sn, cs;
                sincosf(th.v[e], &sn, &cs);
                const float ar = hr.v[e] * cs - hi.v[e] * sn, ai = hr.v[e] * sn + hi.v[e] * cs;
                const float ur = ar - tr.v[e], ui = ai - ti.v[e];
                const float m = sqrtf(ur * ur + ui * ui);
                const float k = m > 0.0f ? -g / m : 0.0f;  // s = gamma - sum m
                const float qpr = k * ur, qpi = k * ui;
                if constexpr (HEAD) {
                    // negatives: a' = t e^{-i theta}, G = dL/da'; positive term as in the tail form
                    const float br = tr.v[e] * cs + ti.v[e] * sn, bi = ti.v[e] * cs - tr.v[e] * sn;
                    dhr.v[e] = qpr * cs + qpi * sn;
                    dhi.v[e] = qpi * cs - qpr * sn;
                    dtr.v[e] = (Gr.v[e] * cs - Gi.v[e] * sn) - qpr;
                    dti.v[e] = (Gi.v[e] * cs + Gr.v[e] * sn) - qpi;
                    dth.v[e] = (qpi * ar - qpr * ai) - (Gi.v[e] * br - Gr.v[e] * bi);
                } else {
                    const float Qr = qpr + Gr.v[e], Qi = qpi + Gi.v[e];
                    dhr.v[e] = Qr * cs + Qi * sn;
                    dhi.v[e] = Qi * cs - Qr * sn;
                    dth.v[e] = Qi * ar - Qr * ai;
                    dtr.v[e] = -qpr;
                    dti.v[e] = -qpi;
                }
            }
            dhr.store(oh + j), dhi.store(oh + half + j);
            dth.store(orr + j);
            dtr.store(ot + j), dti.store(ot + half + j);
        }
    } else if constexpr (MODEL == KGE_TRANSH) {
        const float *w = a.aux + rid * (int64_t)d;
        float *ow = a.occ_w + b * (int64_t)d;
        float sd = 0.0f;
        for (int j = lane * V; j < d; j += kWave * V) {
            const Vec<V> vh = Vec<V>::load(eh + j), vt = Vec<V>::load(et + j), vw = Vec<V>::load(w + j);
#pragma unroll
            for (int e = 0; e < V; ++e) sd += vw.v[e] * (vh.v[e] - vt.v[e]);
        }
        sd = wave_sum(sd);
        float qw = 0.0f, gw = 0.0f;  // q_pos . w and G_q . w
        for (int j = lane * V; j < d; j += kWave * V) {
            const Vec<V> vh = Vec<V>::load(eh + j), vt = Vec<V>::load(et + j), vr = Vec<V>::load(rr + j),
                         vw = Vec<V>::load(w + j);
            const Vec<V> G = ldz<V>(g0, j);
#pragma unroll
            for (int e = 0; e < V; ++e) {
                const float u = ((vh.v[e] - vt.v[e]) + vr.v[e]) - sd * vw.v[e];
                const float q = gs * (P == 1 ? sgn(u) : u);
                qw += q * vw.v[e];
                gw += G.v[e] * vw.v[e];
            }
        }
        qw = wave_sum(qw);
        gw = wave_sum(gw);
        for (int j = lane * V; j < d; j += kWave * V) {
            const Vec<V> vh = Vec<V>::load(eh + j), vt = Vec<V>::load(et + j), vr = Vec<V>::load(rr + j),
                         vw = Vec<V>::load(w + j);
            const Vec<V> G = ldz<V>(g0, j), Gw = ldz<V>(g1, j);
            Vec<V> dh, dt, dr, dw;
#pragma unroll
            for (int e = 0; e < V; ++e) {
                const float d0 = vh.v[e] - vt.v[e];
                const float u = (d0 + vr.v[e]) - sd * vw.v[e];
                const float q = gs * (P == 1 ? sgn(u) : u);
                if constexpr (HEAD) {  // G chains through a = t - r - (w.t) w
                    dr.v[e] = q - G.v[e];
                    dh.v[e] = q - qw * vw.v[e];
                    dt.v[e] = (G.v[e] - gw * vw.v[e]) - (q - qw * vw.v[e]);
                    dw.v[e] = Gw.v[e] - (qw * d0 + sd * q) - gw * vt.v[e];
                } else {
                    const float Q = q + G.v[e];
                    dr.v[e] = Q;
                    dh.v[e] = Q - (qw + gw) * vw.v[e];
                    dt.v[e] = -(q - qw * vw.v[e]);
                    dw.v[e] = Gw.v[e] - (qw * d0 + sd * q) - gw * vh.v[e];
                }
            }
            dh.store(oh + j), dt.store(ot + j), dr.store(orr + j), dw.store(ow + j);
        }
    }
}

template <int MODEL, int P>
static int launch_pos_bwd(const PosBwdArgs &a, bool vec4, bool head, const FusedInsp &fi, hipStream_t st)
{
    const dim3 grid((unsigned)ceil_div(a.B, 4) + (unsigned)fi.blocks), block(256);
    const size_t lds = fi.blocks > 0 ? (size_t)fi.lds_bytes : 0;
    if (head) {
        if (vec4) hipLaunchKernelGGL((bwd_pos_kernel<MODEL, P, 4, true>), grid, block, lds, st, a, fi);
        else hipLaunchKernelGGL((bwd_pos_kernel<MODEL, P, 1, true>), grid, block, lds, st, a, fi);
    } else {
        if (vec4) hipLaunchKernelGGL((bwd_pos_kernel<MODEL, P, 4, false>), grid, block, lds, st, a, fi);
        else hipLaunchKernelGGL((bwd_pos_kernel<MODEL, P, 1, false>), grid, block, lds, st, a, fi);
    }
    KGE_CHECK_LAUNCH();
    return KGE_OK;
}

__global__ void fill_zero_kernel(float *p, int64_t n)
{
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x)
        p[i] = 0.0f;
}

// ---------------------------------------------------------------------------------------
struct BwdPlan {
    int64_t n_occ, nn;
    size_t off_occ_e, off_occ_r, off_occ_w, off_g0, off_g1, off_part_e, off_part_r, off_part_w, total;
};

static size_t up256(size_t x) { return (x + 255) & ~size_t(255); }

static BwdPlan make_bwd_plan(const kge_tables *tab, const kge_batch *bat)
{
    BwdPlan p{};
    const int64_t B = bat->batch, d = tab->dim, rd = tab->rel_dim;
    p.nn = bat->neg ? (B / bat->chunk) * bat->n_neg : 0;
    p.n_occ = 2 * B + p.nn;
    size_t o = 0;
    auto take = [&](int64_t floats) {
        const size_t at = o;
        o += up256(sizeof(float) * (size_t)(floats > 0 ? floats : 1));
        return at;
    };
    p.off_occ_e = take(p.n_occ * d);
    p.off_occ_r = take(B * rd);
    p.off_occ_w = take(tab->model == KGE_TRANSH ? B * d : 0);
    p.off_g0 = take(bat->neg ? B * d : 0);
    p.off_g1 = take(bat->neg && tab->model == KGE_TRANSH ? B * d : 0);
    p.off_part_e = take(seg_partial_floats(p.n_occ, d));
    p.off_part_r = take(seg_partial_floats(B, rd));
    p.off_part_w = take(tab->model == KGE_TRANSH ? seg_partial_floats(B, d) : 0);
    p.total = o;
    return p;
}

// RESCAL with shared negatives (tail mode): the gradient tiles of the dot-product score over the projected
// query rows; g0[B, d] receives dL/dq summed over the chunk's negatives, occ_neg[nn, d] the negatives' rows.
// Called by the grouped backward pass in transr.hip.
int launch_rescal_neg_tiles(const kge_tables *tab, const kge_batch *bat, const float *query, const float *dneg, float *g0,
                            float *occ_neg, hipStream_t st)
{
    const int64_t B = bat->batch, d = tab->dim, n_chunks = B / bat->chunk;
    if (n_chunks >= (1 << 24)) return KGE_ESHAPE;
    const bool vec = rows_vectorizable(tab), vecn = bat->n_neg % 4 == 0 && aligned16(dneg);
    TileArgs a{tab->ent, nullptr, nullptr, bat->h, bat->r, bat->neg, dneg, nullptr, nullptr, nullptr, query, nullptr, nullptr,
               B * bat->n_neg, (int)bat->chunk, (int)bat->n_neg, (int)d, 0, vec ? 1 : 0, vecn ? 1 : 0, (int)n_chunks, 1.0f,
               0, nullptr, nullptr, nullptr, nullptr, nullptr};
    return launch_tiles<KGE_RESCAL, 2>(a, g0, nullptr, occ_neg, n_chunks, pair_sums_valu(tab), FusedInsp{}, st);
}

int launch_transr_bwd(const kge_tables *, const kge_batch *, const kge_saved *, const float *,
                      const kge_grads *, void *, size_t, hipStream_t);
size_t transr_bwd_workspace(const kge_tables *, const kge_batch *);
int launch_transr_neg_bwd(const kge_tables *, const kge_batch *, const kge_saved *, const float *, const float *,
                          const kge_grads *, void *, size_t, hipStream_t);
size_t transr_neg_bwd_workspace(const kge_tables *, const kge_batch *);
int launch_rescal_neg_bwd(const kge_tables *, const kge_batch *, const kge_saved *, const float *, const float *,
                          const kge_grads *, void *, size_t, hipStream_t);

}  // namespace kge

using namespace kge;

extern "C" {

size_t kge_score_bwd_workspace(const kge_tables *tab, const kge_batch *bat)
{
    if (!tab || !bat || bat->batch < 0 || tab->dim <= 0) return 0;
    if (bat->neg && bat->chunk <= 0) return 0;
    if (tab->model == KGE_TRANSR && bat->neg) return transr_neg_bwd_workspace(tab, bat);
    if (tab->model == KGE_TRANSR || tab->model == KGE_RESCAL) return transr_bwd_workspace(tab, bat);
    return make_bwd_plan(tab, bat).total;
}

int kge_score_bwd(const kge_tables *tab, const kge_batch *bat, const kge_saved *saved, const float *dpos,
                  const float *dneg, const kge_grads *grads, void *workspace, size_t workspace_bytes,
                  void *stream)
{
    if (!tab || !bat || !saved || !grads || !tab->ent) return KGE_EINVAL;
    if (bat->batch < 0 || tab->dim <= 0) return KGE_ESHAPE;
    if (bat->batch == 0) return KGE_OK;
    if (!bat->h || !bat->r || !bat->t || !bat->ent_insp || !bat->rel_insp || !grads->ent_rows) return KGE_EINVAL;
    if (bat->neg && (bat->chunk <= 0 || bat->n_neg <= 0 || bat->batch % bat->chunk)) return KGE_ESHAPE;
    hipStream_t st = as_stream(stream);
    KGE_CLEAR_LAUNCH_ERRORS();
    if (tab->model == KGE_TRANSR && bat->neg)
        return launch_transr_neg_bwd(tab, bat, saved, dpos, dneg, grads, workspace, workspace_bytes, st);
    if (tab->model == KGE_RESCAL && bat->neg)
        return launch_rescal_neg_bwd(tab, bat, saved, dpos, dneg, grads, workspace, workspace_bytes, st);
    if (tab->model == KGE_TRANSR || tab->model == KGE_RESCAL)
        return launch_transr_bwd(tab, bat, saved, dpos, grads, workspace, workspace_bytes, st);

    const BwdPlan p = make_bwd_plan(tab, bat);
    if (!workspace || workspace_bytes < p.total) return KGE_EWORKSPACE;
    if (bat->ent_insp->n != p.n_occ || bat->rel_insp->n != bat->batch) return KGE_ESHAPE;
    const int model = tab->model, P = tab->norm_p;
    const bool normed = model == KGE_TRANSE || model == KGE_TRANSH;
    if (normed && P != 1 && P != 2) return KGE_EINVAL;
    if (tab->rel_dim > 0 && !grads->rel_rows) return KGE_EINVAL;
    if (normed && P == 2 && dpos && !saved->pos) return KGE_EINVAL;
    const bool have_neg = bat->neg && dneg;
    if (bat->neg && bat->neg_mode != KGE_NEG_TAIL && bat->neg_mode != KGE_NEG_HEAD) return KGE_EINVAL;
    const bool head = have_neg && bat->neg_mode == KGE_NEG_HEAD;
    if (have_neg) {
        if (normed && P == 2 && !saved->neg) return KGE_EINVAL;
        if (model == KGE_TRANSH && (!saved->side_pos || !saved->side_neg)) return KGE_EINVAL;
        if (model == KGE_ROTATE && !saved->residual) return KGE_EINVAL;  // rotated heads from the forward pass
    }
    if (model == KGE_TRANSH && !grads->aux_rows) return KGE_EINVAL;

    const int64_t B = bat->batch, d = tab->dim;
    char *ws = static_cast<char *>(workspace);
    float *occ_e = reinterpret_cast<float *>(ws + p.off_occ_e);
    float *occ_r = reinterpret_cast<float *>(ws + p.off_occ_r);
    float *occ_w = reinterpret_cast<float *>(ws + p.off_occ_w);
    float *g0 = have_neg ? reinterpret_cast<float *>(ws + p.off_g0) : nullptr;
    float *g1 = have_neg && model == KGE_TRANSH ? reinterpret_cast<float *>(ws + p.off_g1) : nullptr;
    const bool vec = rows_vectorizable(tab);
    bool chained = false;  // the gradient tile kernel wrote the positives' occurrence rows itself
    int rc = KGE_OK;
    // inspection fused into the score kernels' launches: the histogram and the first digit pass
    // rode with the two forward kernels; the last pass rides with the gradient tile kernel, the
    // dedup with the per-positive kernel
    FusedInsp fi_pass{}, fi_dedup{};
    if (bat->fuse_inspection) {
        if (!have_neg || !bat->insp_jobs) return KGE_EINVAL;
        if ((rc = plan_fused_inspection(bat->insp_jobs, 2, 2, &fi_pass))) return rc;
        if ((rc = plan_fused_inspection(bat->insp_jobs, 2, 3, &fi_dedup))) return rc;
    }

    if (have_neg) {
        const int64_t n_chunks = B / bat->chunk;
        if (n_chunks >= (1 << 24)) return KGE_ESHAPE;
        const bool vecn = bat->n_neg % 4 == 0 && aligned16(dneg) && (!saved->neg || aligned16(saved->neg)) &&
                          (!saved->side_neg || aligned16(saved->side_neg));
        const bool dv = pair_sums_valu(tab);
        // the positive chain in the tile kernel's epilogue: see TileArgs::chain
        chained = (model == KGE_DISTMULT || model == KGE_COMPLEX) && !dv && vec && !bat->fuse_inspection;
        TileArgs a{tab->ent, tab->rel, tab->aux, head ? bat->t : bat->h, bat->r, bat->neg, dneg, saved->neg,
                   saved->side_pos, saved->side_neg, model == KGE_ROTATE ? saved->residual : nullptr, nullptr, nullptr,
                   B * bat->n_neg, (int)bat->chunk, (int)bat->n_neg, (int)d, (int)tab->rel_dim, vec ? 1 : 0,
                   vecn ? 1 : 0, (int)n_chunks, head ? -1.0f : 1.0f,
                   chained ? 1 : 0, head ? bat->h : bat->t, dpos, head ? occ_e + B * d : occ_e, head ? occ_e : occ_e + B * d, occ_r};
        float *occ_neg = occ_e + 2 * B * d;
        switch (model) {
        case KGE_TRANSE:
            rc = P == 1 ? launch_tiles<KGE_TRANSE, 1>(a, g0, g1, occ_neg, n_chunks, dv, fi_pass, st)
                        : launch_tiles<KGE_TRANSE, 2>(a, g0, g1, occ_neg, n_chunks, dv, fi_pass, st);
            break;
        case KGE_TRANSH:
            rc = P == 1 ? launch_tiles<KGE_TRANSH, 1>(a, g0, g1, occ_neg, n_chunks, dv, fi_pass, st)
                        : launch_tiles<KGE_TRANSH, 2>(a, g0, g1, occ_neg, n_chunks, dv, fi_pass, st);
            break;
        case KGE_DISTMULT: rc = launch_tiles<KGE_DISTMULT, 2>(a, g0, g1, occ_neg, n_chunks, dv, fi_pass, st); break;
        case KGE_COMPLEX: rc = launch_tiles<KGE_COMPLEX, 2>(a, g0, g1, occ_neg, n_chunks, dv, fi_pass, st); break;
        case KGE_ROTATE: rc = launch_tiles<KGE_ROTATE, 2>(a, g0, g1, occ_neg, n_chunks, dv, fi_pass, st); break;
        case KGE_TRANSF: rc = launch_tiles<KGE_TRANSF, 2>(a, g0, g1, occ_neg, n_chunks, dv, fi_pass, st); break;
        default: return KGE_EUNSUPPORTED;
        }
        timeline_mark(bat->timeline, st, "bwd_tile_kernel");
        if (rc) return rc;
    } else if (p.nn > 0) {
        hipLaunchKernelGGL(fill_zero_kernel, dim3(1024), dim3(256), 0, st, occ_e + 2 * B * d, p.nn * d);
    }

    if (!chained) {
    PosBwdArgs pa{tab->ent, tab->rel, tab->aux, bat->h, bat->r, bat->t, dpos, saved->pos, saved->side_pos,
                  g0, g1, have_neg ? dneg : nullptr, bat->n_neg, occ_e, occ_e + B * d, occ_r, occ_w, B, (int)d,
                  (int)tab->rel_dim};
    switch (model) {
    case KGE_TRANSE:
        rc = P == 1 ? launch_pos_bwd<KGE_TRANSE, 1>(pa, vec, head, fi_dedup, st) : launch_pos_bwd<KGE_TRANSE, 2>(pa, vec, head, fi_dedup, st);
        break;
    case KGE_TRANSH:
        rc = P == 1 ? launch_pos_bwd<KGE_TRANSH, 1>(pa, vec, head, fi_dedup, st) : launch_pos_bwd<KGE_TRANSH, 2>(pa, vec, head, fi_dedup, st);
        break;
    case KGE_DISTMULT: rc = launch_pos_bwd<KGE_DISTMULT, 2>(pa, vec, head, fi_dedup, st); break;
    case KGE_COMPLEX: rc = launch_pos_bwd<KGE_COMPLEX, 2>(pa, vec, head, fi_dedup, st); break;
    case KGE_ROTATE: rc = launch_pos_bwd<KGE_ROTATE, 2>(pa, vec, head, fi_dedup, st); break;
    case KGE_TRANSF: rc = launch_pos_bwd<KGE_TRANSF, 2>(pa, vec, head, fi_dedup, st); break;
    default: return KGE_EUNSUPPORTED;
    }
    timeline_mark(bat->timeline, st, "bwd_pos_kernel");
    if (rc) return rc;
    }

    if (bat->insp_ready && hipStreamWaitEvent(st, reinterpret_cast<hipEvent_t>(bat->insp_ready), 0) != hipSuccess)
        return KGE_ELAUNCH;
    const SegJob jobs[3] = {
        {occ_e, bat->ent_insp, (int)d, grads->ent_rows, reinterpret_cast<float *>(ws + p.off_part_e), false},
        {occ_r, bat->rel_insp, (int)tab->rel_dim, grads->rel_rows, reinterpret_cast<float *>(ws + p.off_part_r), false},
        {occ_w, bat->rel_insp, (int)d, grads->aux_rows, reinterpret_cast<float *>(ws + p.off_part_w), false}};
    return launch_seg_reduce_jobs(jobs, model == KGE_TRANSH ? 3 : 2, st, bat->timeline);
}

}  // extern "C"
