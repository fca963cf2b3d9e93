// Pieces shared by the shared-negative tile kernels (forward and backward): guarded
// 128-bit row loads and the per-model "query" row a_b = f(h_b, r_b) that is formed on
// the fly while a tile is staged, so h and r are gathered inside the consuming kernel.
#pragma once

#include "common.hpp"

#ifndef KGE_TILE_OCC
#define KGE_TILE_OCC 3  // minimum workgroups per CU the tile kernels are compiled for
#endif

namespace kge {

// Four consecutive floats p[j .. j+3], zero where j + e >= lim.  Branch-free: an out-of-range
// request reads p[0] (always a valid row start here) and discards it, so the callers' loads sit
// in one basic block and the compiler can issue them back to back.
template <bool VEC>
__device__ __forceinline__ float4 ld4(const float *p, int j, int lim)
{
    if constexpr (VEC) {  // rows are 16-byte aligned and lim % 4 == 0
        const bool ok = j < lim;
        const float4 v = *reinterpret_cast<const float4 *>(p + (ok ? j : 0));
        return ok ? v : make_float4(0.f, 0.f, 0.f, 0.f);
    } else {
        float4 q;
        const bool k0 = j + 0 < lim, k1 = j + 1 < lim, k2 = j + 2 < lim, k3 = j + 3 < lim;
        const float x0 = p[k0 ? j + 0 : 0], x1 = p[k1 ? j + 1 : 0], x2 = p[k2 ? j + 2 : 0], x3 = p[k3 ? j + 3 : 0];
        q.x = k0 ? x0 : 0.0f;
        q.y = k1 ? x1 : 0.0f;
        q.z = k2 ? x2 : 0.0f;
        q.w = k3 ? x3 : 0.0f;
        return q;
    }
}

__device__ __forceinline__ void st4(float *p, int j, int lim, bool vec, float4 v)
{
    if (vec) {
        if (j < lim) *reinterpret_cast<float4 *>(p + j) = v;
        return;
    }
    if (j + 0 < lim) p[j + 0] = v.x;
    if (j + 1 < lim) p[j + 1] = v.y;
    if (j + 2 < lim) p[j + 2] = v.z;
    if (j + 3 < lim) p[j + 3] = v.w;
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

// sign(u) as a clamp: u * 2^100 clamped to [-1, 1] (exact 0 stays 0; |u| < 2^-100 would give a
// fraction, far below any fp32 residual that is not exactly zero).  The multiply is paid once per
// staged row element instead of once per pair element: scaling by a power of two commutes with
// every fp32 rounding (no overflow: table values times 2^100 stay far below 2^127), so a residual
// formed from rows that carry the factor 2^100 is exactly 2^100 times the residual of the plain
// rows, and its sign is one clamp away.  The L1 tile kernels of TransE / TransH stage their rows
// scaled; sums of |U| and of sign(U) * W are scaled back once per pair, and coefficients that
// multiply a scaled row carry 2^-100.
// Measured alternatives that did not pay (TransH, L1, 16384 x 1024 pairs x 400): clamping
// u * copysign(2^100, g) to [-|g|, |g|] to get g * sign(u) directly (forward 0.92 -> 1.10 ms, gradient
// tiles 1.74 -> 1.86 ms: v_med3_f32 and v_bfi_b32 issue at two thirds of the rate of add / mul / fmac);
// (sign(u) + 1) / 2 as ONE multiply-add with the output clamp, the coefficients' sums taken off once
// per step (one instruction fewer per element, same forward time, gradient tiles 1.74 -> 1.80 ms: a
// v_fma_f32 with a scalar-register operand issues at 60 % of the vector-operand rate, and with the
// factor in a vector register the per-pair bookkeeping ate the gain).
constexpr float kSgnScale = 0x1p100f, kSgnUnscale = 0x1p-100f;
__device__ __forceinline__ float sgn_of_scaled(float U) { return __builtin_amdgcn_fmed3f(U, -1.0f, 1.0f); }
__device__ __forceinline__ float4 scale4(float4 v, float s) { return make_float4(v.x * s, v.y * s, v.z * s, v.w * s); }

// reduction length of the pair kernels: complex pairs for RotatE, floats otherwise
template <int MODEL>
__device__ __forceinline__ int pair_len(int d)
{
    return MODEL == KGE_ROTATE ? d >> 1 : d;
}

// Four consecutive elements (index j .. j+3 of the reduction axis) of the query row.
//   DistMult  q0 = h*r                   ComplEx  q0 = (h o r) laid out [re | im]
//   TransE    q0 = h+r                   RotatE   q0 = Re(h e^{i theta}), q1 = Im(...) (from pq)
//   TransH    q0 = h + r - al*w (al = w.h), q1 = w
//   TransF    q0 = 2h + r: score = (h + r).t' + (t' - r).h = (2h + r).t' - r.h, a dot product with
//             the query plus a constant per positive
//   RESCAL    q0 = E[h] Proj[r], the projected row that the grouped forward pass left in pq:
//             score = (h M_r) . t' needs no projection of the negatives at all
// lim == 0 yields zeros (row outside the tile).
// RotatE takes its query rows from pq, the [B, d] buffer of rotated heads.
//
// Negatives that replace the HEAD use the same pair kernels: score(n, r, t) is the tail-mode
// function of (x, rho, n) with x = t and rho = -r (TransE, TransH, TransF), conj(r) (ComplEx), -theta
// (RotatE, already applied in pq) or r (DistMult).  The caller passes the tail row as `ph` and
// rs = -1; rs multiplies r (its imaginary half for ComplEx), which is exact, so rs = +1
// reproduces the tail-mode arithmetic bit for bit.
template <int MODEL, bool VEC>
__device__ __forceinline__ void load_query(const float *ph, const float *pr, const float *pw, float al,
                                           int j, int lim, int half, float4 &q0, float4 &q1,
                                           const float *pq = nullptr, float rs = 1.0f)
{
    q1 = zero4();
    if constexpr (MODEL == KGE_DISTMULT) {
        q0 = mul4(ld4<VEC>(ph, j, lim), ld4<VEC>(pr, j, lim));
    } else if constexpr (MODEL == KGE_TRANSE) {
        const float4 vh = ld4<VEC>(ph, j, lim), vr = ld4<VEC>(pr, j, lim);
        q0 = make_float4(fmaf(rs, vr.x, vh.x), fmaf(rs, vr.y, vh.y), fmaf(rs, vr.z, vh.z), fmaf(rs, vr.w, vh.w));
    } else if constexpr (MODEL == KGE_TRANSF) {
        const float4 vh = ld4<VEC>(ph, j, lim), vr = ld4<VEC>(pr, j, lim);
        q0 = make_float4(fmaf(rs, vr.x, 2.0f * vh.x), fmaf(rs, vr.y, 2.0f * vh.y), fmaf(rs, vr.z, 2.0f * vh.z),
                         fmaf(rs, vr.w, 2.0f * vh.w));
    } else if constexpr (MODEL == KGE_COMPLEX) {
        float q[4];
        if constexpr (VEC) {  // half % 4 == 0: the four elements sit on one side of the re|im split
            const bool re = j < half;
            const int i = re ? j : j - half;
            const int l2 = lim ? half : 0;
            const float4 hr = ld4<true>(ph, i, l2), hi = ld4<true>(ph + half, i, l2);
            const float4 rr = ld4<true>(pr, i, l2);
            float4 ri = ld4<true>(pr + half, i, l2);
            ri = make_float4(rs * ri.x, rs * ri.y, rs * ri.z, rs * ri.w);
            q[0] = re ? hr.x * rr.x - hi.x * ri.x : hr.x * ri.x + hi.x * rr.x;
            q[1] = re ? hr.y * rr.y - hi.y * ri.y : hr.y * ri.y + hi.y * rr.y;
            q[2] = re ? hr.z * rr.z - hi.z * ri.z : hr.z * ri.z + hi.z * rr.z;
            q[3] = re ? hr.w * rr.w - hi.w * ri.w : hr.w * ri.w + hi.w * rr.w;
        } else {
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const int jj = j + e;
                const bool ok = jj < lim;
                const int i = ok ? (jj < half ? jj : jj - half) : 0;
                const float hr = ph[i], hi = ph[i + half], rr = pr[i], ri = rs * pr[i + half];
                q[e] = ok ? (jj < half ? hr * rr - hi * ri : hr * ri + hi * rr) : 0.0f;
            }
        }
        q0 = make_float4(q[0], q[1], q[2], q[3]);
    } else if constexpr (MODEL == KGE_RESCAL) {
        q0 = ld4<VEC>(pq, j, lim);
    } else if constexpr (MODEL == KGE_ROTATE) {
        // the rotated head h e^{i theta} was written by the positive kernel ([re | im] row pq):
        // a plain load here instead of a sincos per element in every tile that needs the row
        q0 = ld4<VEC>(pq, j, lim);
        q1 = ld4<VEC>(pq + half, j, lim);
    } else if constexpr (MODEL == KGE_TRANSH) {
        const float4 vw = ld4<VEC>(pw, j, lim);
        const float4 vh = ld4<VEC>(ph, j, lim), vr = ld4<VEC>(pr, j, lim);
        q1 = vw;
        q0 = make_float4(fmaf(rs, vr.x, vh.x) - al * vw.x, fmaf(rs, vr.y, vh.y) - al * vw.y,
                         fmaf(rs, vr.z, vh.z) - al * vw.z, fmaf(rs, vr.w, vh.w) - al * vw.w);
    } else {
        q0 = zero4();
    }
}

// ---- the same in two steps ---------------------------------------------------------------------
// A tile kernel that prefetches the next block of rows while it computes on the current one only
// overlaps the two if nothing touches the loaded registers before the compute: any arithmetic
// on them (h * r, the zero fill of a tail) makes the compiler wait for the loads where they are
// issued.  load_query_raw() therefore only loads -- clamped to a valid address, no select, no
// arithmetic -- and combine_query() forms the query row when the block is written to LDS.
template <bool VEC>
__device__ __forceinline__ float4 ld4_raw(const float *p, int j, int lim)
{
    if constexpr (VEC) {  // rows are 16-byte aligned and lim % 4 == 0
        return *reinterpret_cast<const float4 *>(p + (j < lim ? j : 0));
    } else {
        return make_float4(p[j + 0 < lim ? j + 0 : 0], p[j + 1 < lim ? j + 1 : 0], p[j + 2 < lim ? j + 2 : 0],
                           p[j + 3 < lim ? j + 3 : 0]);
    }
}

// zero the elements at or beyond lim (the whole quad when VEC)
template <bool VEC>
__device__ __forceinline__ float4 mask4(float4 v, int j, int lim)
{
    if constexpr (VEC) return j < lim ? v : make_float4(0.f, 0.f, 0.f, 0.f);
    return make_float4(j + 0 < lim ? v.x : 0.0f, j + 1 < lim ? v.y : 0.0f, j + 2 < lim ? v.z : 0.0f,
                       j + 3 < lim ? v.w : 0.0f);
}

template <int MODEL>
constexpr int query_raw_count()
{
    return MODEL == KGE_COMPLEX ? 4 : (MODEL == KGE_TRANSH ? 3 : 2);
}

template <int MODEL, bool VEC, int N>
__device__ __forceinline__ void load_query_raw(const float *ph, const float *pr, const float *pw, const float *pq,
                                               int j, int lim, int half, float4 (&raw)[N])
{
    static_assert(N == query_raw_count<MODEL>(), "raw operand count");
    if constexpr (MODEL == KGE_DISTMULT || MODEL == KGE_TRANSE || MODEL == KGE_TRANSF) {
        raw[0] = ld4_raw<VEC>(ph, j, lim);
        raw[1] = ld4_raw<VEC>(pr, j, lim);
    } else if constexpr (MODEL == KGE_COMPLEX) {
        if constexpr (VEC) {  // half % 4 == 0: the four elements sit on one side of the re|im split
            const int i = j < half ? j : j - half;
            const int l2 = lim ? half : 0;
            raw[0] = ld4_raw<true>(ph, i, l2), raw[1] = ld4_raw<true>(ph + half, i, l2);
            raw[2] = ld4_raw<true>(pr, i, l2), raw[3] = ld4_raw<true>(pr + half, i, l2);
        } else {
            float v[4][4];
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const int jj = j + e;
                const int i = jj < lim ? (jj < half ? jj : jj - half) : 0;
                v[0][e] = ph[i], v[1][e] = ph[i + half], v[2][e] = pr[i], v[3][e] = pr[i + half];
            }
#pragma unroll
            for (int n = 0; n < 4; ++n) raw[n] = make_float4(v[n][0], v[n][1], v[n][2], v[n][3]);
        }
    } else if constexpr (MODEL == KGE_RESCAL) {
        raw[0] = ld4_raw<VEC>(pq, j, lim);
        raw[1] = raw[0];
    } else if constexpr (MODEL == KGE_ROTATE) {
        raw[0] = ld4_raw<VEC>(pq, j, lim);
        raw[1] = ld4_raw<VEC>(pq + half, j, lim);
    } else if constexpr (MODEL == KGE_TRANSH) {
        raw[0] = ld4_raw<VEC>(pw, j, lim);
        raw[1] = ld4_raw<VEC>(ph, j, lim);
        raw[2] = ld4_raw<VEC>(pr, j, lim);
    }
}

// The query row from its raw operands (same j, lim, half, rs as load_query; same arithmetic).
template <int MODEL, bool VEC, int N>
__device__ __forceinline__ void combine_query(const float4 (&raw)[N], float al, int j, int lim, int half, float rs,
                                              float4 &q0, float4 &q1)
{
    q1 = zero4();
    if constexpr (MODEL == KGE_DISTMULT) {
        q0 = mask4<VEC>(mul4(raw[0], raw[1]), j, lim);
    } else if constexpr (MODEL == KGE_TRANSE) {
        const float4 vh = raw[0], vr = raw[1];
        q0 = mask4<VEC>(make_float4(fmaf(rs, vr.x, vh.x), fmaf(rs, vr.y, vh.y), fmaf(rs, vr.z, vh.z), fmaf(rs, vr.w, vh.w)),
                        j, lim);
    } else if constexpr (MODEL == KGE_TRANSF) {
        const float4 vh = raw[0], vr = raw[1];
        q0 = mask4<VEC>(make_float4(fmaf(rs, vr.x, 2.0f * vh.x), fmaf(rs, vr.y, 2.0f * vh.y), fmaf(rs, vr.z, 2.0f * vh.z),
                                    fmaf(rs, vr.w, 2.0f * vh.w)),
                        j, lim);
    } else if constexpr (MODEL == KGE_COMPLEX) {
        const float hr[4] = {raw[0].x, raw[0].y, raw[0].z, raw[0].w}, hi[4] = {raw[1].x, raw[1].y, raw[1].z, raw[1].w};
        const float rr[4] = {raw[2].x, raw[2].y, raw[2].z, raw[2].w};
        const float ri[4] = {rs * raw[3].x, rs * raw[3].y, rs * raw[3].z, rs * raw[3].w};
        float q[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const int jj = VEC ? j : j + e;  // VEC: one side of the split for the whole quad
            const float v = jj < half ? hr[e] * rr[e] - hi[e] * ri[e] : hr[e] * ri[e] + hi[e] * rr[e];
            q[e] = jj < lim ? v : 0.0f;
        }
        q0 = make_float4(q[0], q[1], q[2], q[3]);
    } else if constexpr (MODEL == KGE_RESCAL) {
        q0 = mask4<VEC>(raw[0], j, lim);
    } else if constexpr (MODEL == KGE_ROTATE) {
        q0 = mask4<VEC>(raw[0], j, lim);
        q1 = mask4<VEC>(raw[1], j, lim);
    } else if constexpr (MODEL == KGE_TRANSH) {
        const float4 vw = raw[0], vh = raw[1], vr = raw[2];
        q1 = mask4<VEC>(vw, j, lim);
        q0 = mask4<VEC>(make_float4(fmaf(rs, vr.x, vh.x) - al * vw.x, fmaf(rs, vr.y, vh.y) - al * vw.y,
                                    fmaf(rs, vr.z, vh.z) - al * vw.z, fmaf(rs, vr.w, vh.w) - al * vw.w),
                        j, lim);
    } else {
        q0 = zero4();
    }
}

// XCD-aware tile placement.  The 256 CUs sit in 8 XCDs with one L2 each, and consecutive
// workgroup ids of a 1-D grid go to consecutive XCDs.  All tiles of one chunk share that
// chunk's positive and negative rows, so they are steered to one XCD: every gathered row is
// then fetched from HBM by a single L2 instead of by up to eight.  With fewer than 8 chunks a
// chunk's tiles are dealt round-robin to 8 / n_chunks XCDs so that no XCD stays idle.
// Returns false for the padding ids of the grid (see xcd_grid).
constexpr int kXcds = 8;
__host__ __device__ inline int xcd_split(int n_chunks) { return n_chunks >= kXcds ? 1 : kXcds / n_chunks; }
__device__ __forceinline__ bool xcd_tile(int lid, int tiles_x, int tiles_y, int n_chunks, int &c, int &ty, int &tx)
{
    const int per = tiles_x * tiles_y;
    const int split = xcd_split(n_chunks);
    const int per_v = (per + split - 1) / split;  // tiles of one virtual chunk
    const int xcd = lid % kXcds, k = lid / kXcds;
    const int vc = (k / per_v) * kXcds + xcd;      // virtual chunk = (chunk, residue of the tile id)
    c = vc / split;
    const int t = (k % per_v) * split + vc % split;
    ty = t / tiles_x;
    tx = t % tiles_x;
    return c < n_chunks && t < per;
}
inline unsigned xcd_grid(int64_t tiles_x, int64_t tiles_y, int64_t n_chunks)
{
    const int64_t split = xcd_split((int)n_chunks), per = tiles_x * tiles_y;
    return (unsigned)(kXcds * ceil_div(n_chunks * split, kXcds) * ceil_div(per, split));
}

inline bool rows_vectorizable(const kge_tables *tab)
{
    const bool complex_rows = tab->model == KGE_COMPLEX || tab->model == KGE_ROTATE;
    return tab->dim % (complex_rows ? 8 : 4) == 0 && aligned16(tab->ent) &&
           (!tab->rel || aligned16(tab->rel)) && (!tab->aux || aligned16(tab->aux));
}

}  // namespace kge
