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
#include "inspector_mid.hpp"
#include "seg_reduce.hpp"

namespace kge {

typedef float floatx4 __attribute__((ext_vector_type(4)));

constexpr int kTM = 32;          // triples per tile
#ifndef KGE_TR_RING
#define KGE_TR_RING 3
#endif
#ifndef KGE_TR_OCC
#define KGE_TR_OCC 3
#endif
constexpr int kRing = KGE_TR_RING;  // supersteps of B operands kept in flight per wave
#ifndef KGE_TR_DM_RING
#define KGE_TR_DM_RING 4
#endif
constexpr int kDmRing = KGE_TR_DM_RING;  // the same for the dM kernel's operand stages

constexpr int kThin = 4;            // a group's last tile with at most this many triples takes the thin path
constexpr int kThinRing = 8;        // 128-bit projection loads in flight per thread on the thin path
constexpr int kMaxDimMfma = 1024;
// Dynamic LDS a grouped kernel may ask for: a CU of gfx950 has 160 KB, a few hundred bytes of
// which the kernels' static arrays take.  The 32 x d left-operand tile needs 66.5 KB at d = 512
// and 129 KB at d = 1024 (then one workgroup per CU).
constexpr size_t kMaxGemmLds = 158 * 1024;

int launch_score_pos(const kge_tables *, const kge_batch *, float *, float *, float *, hipStream_t);

// ---- tile plan: one entry per (relation group, block of `tile` sorted positions) -----------
struct TilePlan {
    int32_t *num_tiles;  // [1]
    int32_t *tile_seg;   // [max_tiles] group (unique-relation index)
    int32_t *tile_p0;    // [max_tiles] first sorted position
    int32_t *tile_end;   // [max_tiles] end of the tile's group in sorted positions (GEMM plan only, else null)
    int32_t *tile_rid;   // [max_tiles] relation id of the group (GEMM plan only, else null)
    // groups longer than one tile ("split" groups, used by the dM kernel): every tile of such
    // a group writes a partial result to slot tile_part[tile]; -1 for unsplit groups
    int32_t *tile_part;   // [max_tiles] or null
    int32_t *num_split;   // [1]
    int32_t *split_seg;   // [max_split] group of the split
    int32_t *split_first; // [max_split] first partial slot
    int32_t *split_cnt;   // [max_split] number of partial slots
    // Chunked plan only: the dM kernel's work as compact lists.  How many entries a batch has is only
    // known on the device, and a grid sized for the worst case (one chunk per possible relation, seven row
    // blocks per chunk, one thin workgroup per possible relation: eleven thousand workgroups for a few
    // hundred items) spends 25 us merely being dispatched: the kernel runs kDmWgs workgroups that stride
    // over the lists instead.
    int32_t *num_items;   // [2] long items (from the front of item_*), small-group items (from the back)
    int32_t *item_tile, *item_blk;  // [max_items] (tile, 32-row block), or (tile, -1) = every row block of a small group
    int32_t *num_thin;    // [1]
    int32_t *thin_g;      // [max_tiles] groups of at most kThin triples (no tiles)
    int max_items;
};

#ifndef KGE_TR_DM_WGS
#define KGE_TR_DM_WGS (3 * 256)
#endif
constexpr int kDmWgs = KGE_TR_DM_WGS;  // workgroups of a dM launch: three per CU, what its registers allow

// Inclusive scan over the 1024 threads of the block: shuffle scan inside each wave, then the 16
// wave totals are scanned by every wave for itself (two barriers in all).
__device__ int block_inclusive_scan_1024(int v, int *s_scan)
{
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
#pragma unroll
    for (int o = 1; o < 64; o <<= 1) {
        const int u = __shfl_up(v, o, kWave);
        if (lane >= o) v += u;
    }
    __syncthreads();  // s_scan may still be read from the previous call
    if (lane == 63) s_scan[wave] = v;
    __syncthreads();
    int before = 0;
#pragma unroll
    for (int w = 0; w < 16; ++w) before += w < wave ? s_scan[w] : 0;
    return v + before;
}

// One workgroup per plan: block 0 builds `plan0` with tiles of `tile0` positions (the GEMM plan), block 1
// (when launched) `plan1`, the chunked plan of the dM kernel: chunks of `tile1` positions, `nib` row blocks per
// chunk, groups of at most `small_max` triples as one item.
__global__ __launch_bounds__(1024) void transr_plan_kernel(const int32_t *num_unique, const int32_t *seg_offsets,
                                                          const int64_t *unique_ids, TilePlan plan0, int tile0,
                                                          TilePlan plan1, int tile1, int nib, int small_max)
{
    const bool chunked = blockIdx.x != 0;
    const TilePlan &plan = chunked ? plan1 : plan0;
    const int tile = chunked ? tile1 : tile0;
    __shared__ int s_scan[1024];
    __shared__ int s_carry[6];  // tiles, split slots, splits, thin groups, long items, small items
    const int U = num_unique[0];
    if (threadIdx.x < 6) s_carry[threadIdx.x] = 0;
    __syncthreads();
    for (int base = 0; base < U; base += 1024) {
        const int g = base + threadIdx.x;
        int s0 = 0, s1 = 0, cnt = 0, rid = 0, thin = 0, n_long = 0, n_small = 0;
        if (g < U) {
            s0 = seg_offsets[g], s1 = seg_offsets[g + 1];
            rid = (int)unique_ids[g];
            const int n = s1 - s0;
            cnt = (n + tile - 1) / tile;
            if (chunked) {  // groups of at most kThin triples have no tiles: thin work writes those
                thin = n <= kThin ? 1 : 0;
                if (thin) cnt = 0;
                else if (n <= small_max) n_small = 1;
                else n_long = cnt * nib;
            }
        }
        const int inc_t = block_inclusive_scan_1024(cnt, s_scan);
        const int start = s_carry[0] + inc_t - cnt;
        int pstart = -1, inc_p = 0, inc_s = 0, inc_th = 0, inc_l = 0, inc_m = 0;
        if (chunked) {
            const int pc = cnt > 1 ? cnt : 0, sg = cnt > 1 ? 1 : 0;
            inc_p = block_inclusive_scan_1024(pc, s_scan);
            inc_s = block_inclusive_scan_1024(sg, s_scan);
            inc_th = block_inclusive_scan_1024(thin, s_scan);
            inc_l = block_inclusive_scan_1024(n_long, s_scan);
            inc_m = block_inclusive_scan_1024(n_small, s_scan);
            if (sg) {
                pstart = s_carry[1] + inc_p - pc;
                const int si = s_carry[2] + inc_s - 1;
                plan.split_seg[si] = g;
                plan.split_first[si] = pstart;
                plan.split_cnt[si] = cnt;
            }
            if (thin) plan.thin_g[s_carry[3] + inc_th - 1] = g;
            if (n_small) {  // from the back of the list
                const int at = plan.max_items - 1 - (s_carry[5] + inc_m - 1);
                plan.item_tile[at] = start, plan.item_blk[at] = -1;
            }
            int at = s_carry[4] + inc_l - n_long;
            for (int q = 0; q < (n_long ? cnt : 0); ++q)
                for (int ib = 0; ib < nib; ++ib, ++at) plan.item_tile[at] = start + q, plan.item_blk[at] = ib;
        }
        for (int q = 0; q < cnt; ++q) {
            plan.tile_seg[start + q] = g;
            plan.tile_p0[start + q] = s0 + q * tile;
            if (plan.tile_end) plan.tile_end[start + q] = s1, plan.tile_rid[start + q] = rid;
            if (plan.tile_part) plan.tile_part[start + q] = pstart >= 0 ? pstart + q : -1;
        }
        __syncthreads();
        if (threadIdx.x == 1023) {
            s_carry[0] += inc_t;
            s_carry[1] += inc_p, s_carry[2] += inc_s, s_carry[3] += inc_th, s_carry[4] += inc_l, s_carry[5] += inc_m;
        }
        __syncthreads();
    }
    if (threadIdx.x == 0) {
        plan.num_tiles[0] = s_carry[0];
        if (chunked) {
            plan.num_split[0] = s_carry[2];
            plan.num_thin[0] = s_carry[3];
            plan.num_items[0] = s_carry[4], plan.num_items[1] = s_carry[5];
        }
    }
}

// Where the backward kernels take their operands from when no kernel has written them out.  Sorted
// position p of the relation order names the triple b = perm[p]; its upstream row is
//   TransR  q = c * phi(resid[b]),  c = dpos[b] and phi = sign (L1), or c = dpos[b] / pos[b] and phi = identity (L2)
//   RESCAL  q = c * E[t[b]],        c = dpos[b]
// and its left operand x = E[h[b]] - E[t[b]] (TransR) or E[h[b]] (RESCAL).  The dX and dM kernels form
// both while they stage their tiles: the few scalars per row ride in the index chain the tiles walk
// anyway, and nothing of size B x d is written to memory and read back in between.
struct BwdSrc {
    const float *ent, *resid, *dpos, *spos;
    const int64_t *h, *t;
    const int32_t *perm;
    int norm_p, rescal;
    float *occ_v;  // RESCAL: [B, d] occurrence rows of the tails, g * (E[h] Proj[r]); written by the dX kernel
    int unit;      // non-zero: every coefficient is 1 (the rows phi(residual) Proj^T themselves: GemmArgs::back)
};

struct RowMeta {
    int b;         // triple
    float coef;    // c above
    int64_t qoff;  // offset of the row phi() is applied to, in qbase() floats
    int64_t xh, xt;
};

__device__ __forceinline__ const float *bwd_qbase(const BwdSrc &s) { return s.rescal ? s.ent : s.resid; }

__device__ __forceinline__ RowMeta bwd_row_meta(const BwdSrc &s, int p, int d)
{
    RowMeta m;
    m.b = s.perm[p];
    const float g = s.unit ? 1.0f : (s.dpos ? s.dpos[m.b] : 0.0f);
    m.coef = g;
    if (!s.unit && !s.rescal && s.norm_p == 2) {
        const float sc = s.spos[m.b];
        m.coef = sc > 0.0f ? g / sc : 0.0f;
    }
    m.xh = s.h[m.b], m.xt = s.t[m.b];
    m.qoff = s.rescal ? m.xt * d : (int64_t)m.b * d;
    return m;
}

__device__ __forceinline__ float4 sgn4(float4 v) { return make_float4(sgn(v.x), sgn(v.y), sgn(v.z), sgn(v.w)); }
__device__ __forceinline__ float4 scaled4(float c, float4 v) { return make_float4(c * v.x, c * v.y, c * v.z, c * v.w); }

// ---- grouped GEMM tile: Y[32 x d] = X[32 x d] * M (or * M^T) -----------------------------
struct GemmArgs {
    const float *ent, *rel, *proj;
    const int64_t *h, *r, *t;
    const int32_t *perm, *seg_offsets, *num_unique;
    const int64_t *unique_ids;
    TilePlan plan;
    const float *xs;  // TRANSPOSED pass: left operand rows in sorted order [B, d]; null: formed from `src`.
                      // RESCAL forward (MODE 1), optional: the rows x in sorted order instead of E[h]
    const float *rs;  // list pass (MODE 3): factor of the relation row per list row (+1, -1 or 0)
    float *pos;       // forward: [B] scores (nullable)
    float *resid;     // forward: [B, d] rows y (nullable)
    float *occ_h, *occ_t;  // backward-dX: [B, d] each (occ_t nullable)
    int d, norm_p;
    int thin_groups;       // upper bound of the number of relation groups = trailing thin workgroups
    int max_tiles;         // leading workgroups: planned tiles
    BwdSrc src;            // TRANSPOSED pass without xs
    float *back;           // forward TransR, optional: [B, d] rows phi(y_b) Proj^T, a second sweep of the tile / thin group
};

// ---- thin path: the last <= kThin triples of a relation group ---------------------------------
// More than half of the distinct relations of a Zipf-distributed batch occur only a few times.
// Such a tile is a matrix-vector product that streams the whole 4*d*d-byte projection for a
// handful of rows: what matters is the number of bytes in flight, not the matrix cores.  The
// thin kernels walk the projection as one contiguous array of 128-bit loads with kThinRing loads
// per thread in flight and keep the (up to four) left-hand rows in LDS / registers.

struct ThinTile {
    int rows, p0;
};

// workgroup g looks at group g; returns rows == 0 when the group has no thin tail tile
__device__ __forceinline__ ThinTile thin_tile_of_group(const int32_t *num_unique, const int32_t *seg_offsets, int g)
{
    ThinTile t{0, 0};
    if (g >= num_unique[0]) return t;
    const int s0 = seg_offsets[g], s1 = seg_offsets[g + 1];
    const int rows = (s1 - s0 - 1) % kTM + 1;
    if (rows > kThin) return t;
    t.rows = rows;
    t.p0 = s1 - rows;
    return t;
}

// Y[r][:] = X[r][:] * M for the r < rows <= 4 triples of the tile (MODE 0 TransR, MODE 1 RESCAL,
// MODE 3 list rows: x = E[h] - E[t] with t = -1 standing for no row, y = x M + rs R[r], no score).
// Thread (phase, cq) owns the four columns 4 cq .. 4 cq + 3 and the projection rows
// k = phase, phase + P, ... (P = 256 / (d / 4) phases): consecutive threads read consecutive
// 16-byte pieces of the projection.  The phases are summed through LDS in a fixed order.
template <int MODE>
__device__ __forceinline__ void transr_thin_fwd_body(const GemmArgs &a, float *lds, int g)
{
    const ThinTile tt = thin_tile_of_group(a.num_unique, a.seg_offsets, g);
    const int rows = tt.rows;
    if (rows == 0) return;
    const int d = a.d, nq4 = d >> 2, tid = threadIdx.x;
    const int P = 256 / nq4;
    const int kcap = ((d + P - 1) / P + kThinRing) * P;  // k range the prefetch can name
    float4 *sXT = reinterpret_cast<float4 *>(lds);        // [kcap] x[0..3][k]
    float4 *sRed = sXT + kcap;                             // [P][4][nq4]
    float *sPart = reinterpret_cast<float *>(sRed + P * 4 * nq4);  // [4][nq4]
    __shared__ int s_b[kThin];
    __shared__ int64_t s_h[kThin], s_t[kThin];
    __shared__ float s_rs[kThin];
    const int64_t rid = a.unique_ids[g];
    const float4 *M4 = reinterpret_cast<const float4 *>(a.proj + rid * (int64_t)d * d);
    // The first kThinRing loads of the projection stream only depend on the relation: they are
    // requested before the rows are staged and fly during the index chain and the row gathers.
    const int cq = tid % nq4, ph = tid / nq4;
    const bool active = ph < P;
    // x is zero for k >= d, so a clamped (always valid) address needs no branch; threads beyond the
    // last phase read what phase P - 1 reads and compute nothing
    const int phc = active ? ph : P - 1;
    auto loadm = [&](int k) { return M4[(int64_t)(k < d ? k : d - 1) * nq4 + cq]; };
    float4 ring[kThinRing];
#pragma unroll
    for (int u = 0; u < kThinRing; ++u) ring[u] = loadm(phc + P * u);
    __builtin_amdgcn_sched_barrier(0);
    if (tid < kThin) {
        const int b = tid < rows ? (MODE == 3 ? tt.p0 + tid : a.perm[tt.p0 + tid]) : (MODE == 3 ? tt.p0 : 0);
        s_b[tid] = b;
        s_h[tid] = a.h[b];
        s_t[tid] = a.t[b];
        if constexpr (MODE == 3) s_rs[tid] = a.rs[b];
    }
    for (int k = tid; k < kcap; k += 256) sXT[k] = make_float4(0.f, 0.f, 0.f, 0.f);
    __syncthreads();
    for (int f = tid; f < rows * nq4; f += 256) {
        const int r = f / nq4, k4 = (f % nq4) * 4;
        float4 v = (MODE == 1 && a.xs) ? *reinterpret_cast<const float4 *>(a.xs + (int64_t)(tt.p0 + r) * d + k4)
                                       : *reinterpret_cast<const float4 *>(a.ent + s_h[r] * (int64_t)d + k4);
        if constexpr (MODE == 0) {
            const float4 u = *reinterpret_cast<const float4 *>(a.ent + s_t[r] * (int64_t)d + k4);
            v = make_float4(v.x - u.x, v.y - u.y, v.z - u.z, v.w - u.w);
        }
        if constexpr (MODE == 3) {
            if (s_t[r] >= 0) {
                const float4 u = *reinterpret_cast<const float4 *>(a.ent + s_t[r] * (int64_t)d + k4);
                v = make_float4(v.x - u.x, v.y - u.y, v.z - u.z, v.w - u.w);
            }
        }
        float *col = reinterpret_cast<float *>(sXT + k4) + r;
        col[0] = v.x, col[4] = v.y, col[8] = v.z, col[12] = v.w;
    }
    __syncthreads();

    float4 acc[4];
#pragma unroll
    for (int r = 0; r < 4; ++r) acc[r] = make_float4(0.f, 0.f, 0.f, 0.f);
    if (active) {
        for (int k0 = ph; k0 < d; k0 += P * kThinRing) {
#pragma unroll
            for (int u = 0; u < kThinRing; ++u) {
                const int k = k0 + P * u;
                float4 m = ring[u];
                ring[u] = loadm(k + P * kThinRing);
                const float4 x = sXT[k];  // zero beyond d
                if (k >= d) m = make_float4(0.f, 0.f, 0.f, 0.f);  // keeps 0 * inf out
                const float xr[4] = {x.x, x.y, x.z, x.w};
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    acc[r].x = fmaf(xr[r], m.x, acc[r].x);
                    acc[r].y = fmaf(xr[r], m.y, acc[r].y);
                    acc[r].z = fmaf(xr[r], m.z, acc[r].z);
                    acc[r].w = fmaf(xr[r], m.w, acc[r].w);
                }
            }
        }
#pragma unroll
        for (int r = 0; r < 4; ++r) sRed[(ph * 4 + r) * nq4 + cq] = acc[r];
    }
    __syncthreads();
    for (int f = tid; f < rows * nq4; f += 256) {
        const int r = f / nq4, q = f % nq4;
        float4 y = sRed[r * nq4 + q];
        for (int pp = 1; pp < P; ++pp) {
            const float4 v = sRed[(pp * 4 + r) * nq4 + q];
            y.x += v.x, y.y += v.y, y.z += v.z, y.w += v.w;
        }
        float sum = 0.0f;
        if constexpr (MODE == 0) {
            const float4 rv = *reinterpret_cast<const float4 *>(a.rel + rid * (int64_t)d + 4 * q);
            y.x += rv.x, y.y += rv.y, y.z += rv.z, y.w += rv.w;
            sum = a.norm_p == 1 ? fabsf(y.x) + fabsf(y.y) + fabsf(y.z) + fabsf(y.w)
                                : y.x * y.x + y.y * y.y + y.z * y.z + y.w * y.w;
        } else if constexpr (MODE == 3) {
            const float4 rv = *reinterpret_cast<const float4 *>(a.rel + rid * (int64_t)d + 4 * q);
            const float f = s_rs[r];  // +-1 or 0: the products are exact, the sum rounds as in MODE 0
            y.x += f * rv.x, y.y += f * rv.y, y.z += f * rv.z, y.w += f * rv.w;
        } else {
            const float4 tv = *reinterpret_cast<const float4 *>(a.ent + s_t[r] * (int64_t)d + 4 * q);
            sum = y.x * tv.x + y.y * tv.y + y.z * tv.z + y.w * tv.w;
        }
        if (a.resid) *reinterpret_cast<float4 *>(a.resid + (int64_t)s_b[r] * d + 4 * q) = y;
        sPart[r * nq4 + q] = sum;
    }
    if (!a.pos) return;
    __syncthreads();
    const int wave = tid >> 6, lane = tid & 63;
    if (wave < rows) {  // wave r adds row r's column sums in a fixed order
        float s = 0.0f;
        for (int q = lane; q < nq4; q += kWave) s += sPart[wave * nq4 + q];
        s = wave_sum(s);
        if (lane == 0) a.pos[s_b[wave]] = (MODE == 0 && a.norm_p == 2) ? sqrtf(s) : s;
    }
}

static size_t thin_fwd_lds_bytes(int d)
{
    const int nq4 = d / 4, P = 256 / nq4;
    const int kcap = ((d + P - 1) / P + kThinRing) * P;
    return sizeof(float4) * ((size_t)kcap + (size_t)P * 4 * nq4) + sizeof(float) * 4 * (size_t)nq4;
}

// Sum over the 16 lanes of a DPP row; every lane of the row ends up with the total.
__device__ __forceinline__ float row16_sum(float v)
{
    v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0xB1, 0xF, 0xF, true));   // quad_perm [1,0,3,2]
    v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x4E, 0xF, 0xF, true));   // quad_perm [2,3,0,1]
    v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x141, 0xF, 0xF, true));  // row_half_mirror
    v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x140, 0xF, 0xF, true));  // row_mirror
    return v;
}

// dX for a thin tile: Y[r][j] = sum_k Q[r][k] M[j][k].  Sixteen lanes share one projection row j:
// lane i of the group reads the k-quads i, i + 16, ... (each load instruction covers 256
// contiguous bytes of the row) against its quads of the (up to four) Q rows held in registers,
// and the sixteen partial sums are added with four DPP steps, no LDS and no barrier in the loop.
// A wave works on four rows at a time, the four waves interleave; NS = quads per lane.  Rows wider
// than 64 NS floats are covered in several passes over k-chunks that add into the staged result.
template <int NS>
__device__ __forceinline__ void transr_thin_dx_body(const GemmArgs &a, float *sY, int g)  // sY: [4][d]
{
    const ThinTile tt = thin_tile_of_group(a.num_unique, a.seg_offsets, g);
    const int rows = tt.rows;
    if (rows == 0) return;
    constexpr int R = 8 / NS;  // row groups in flight per wave: R * NS loads per lane
    const int d = a.d, nq4 = d >> 2, tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int li = lane & 15, sub = lane >> 4;
    __shared__ int s_b[kThin];
    const bool derived = a.xs == nullptr;  // the upstream rows are formed here (BwdSrc)
    // (the same addresses in every lane: the compiler turns these into scalar loads)
    const float *qrow[4];
    float qcoef[4], qg[4];
#pragma unroll
    for (int r = 0; r < 4; ++r) {
        const int p = tt.p0 + (r < rows ? r : 0);
        if (derived) {
            const RowMeta m = bwd_row_meta(a.src, p, d);
            qrow[r] = bwd_qbase(a.src) + m.qoff, qcoef[r] = m.coef, qg[r] = a.src.dpos ? a.src.dpos[m.b] : 0.0f;
            if (tid == r) s_b[r] = m.b;
        } else {
            qrow[r] = a.xs + (int64_t)p * d, qcoef[r] = 1.0f, qg[r] = 0.0f;
            if (tid == r) s_b[r] = r < rows ? (a.perm ? a.perm[p] : p) : 0;  // no perm: rows stay in sorted order
        }
    }
    const bool sign_rows = derived && !a.src.rescal && a.src.norm_p == 1;
    const int64_t rid = a.unique_ids[g];
    const float4 *M4 = reinterpret_cast<const float4 *>(a.proj + rid * (int64_t)d * d);
    const int jfirst = 4 * wave + sub;  // row of (step i, wave, sub): j = 16 i + 4 wave + sub
    for (int c0 = 0; c0 < nq4; c0 += 16 * NS) {  // k-chunk of 16 NS quads
        float4 q[NS][4];
        int qc[NS];
#pragma unroll
        for (int s = 0; s < NS; ++s) {
            const int c = c0 + li + 16 * s;
            qc[s] = c < nq4 ? c : 0;
#pragma unroll
            for (int r = 0; r < 4; ++r) {  // zero beyond the row and beyond `rows`: clamped loads then add nothing
                q[s][r] = (c < nq4 && r < rows) ? *reinterpret_cast<const float4 *>(qrow[r] + 4 * c)
                                                : make_float4(0.f, 0.f, 0.f, 0.f);
                if (derived) q[s][r] = scaled4(qcoef[r], sign_rows ? sgn4(q[s][r]) : q[s][r]);
            }
        }
        auto loadrow = [&](int j, float4 *dst) {
            const int64_t base = (int64_t)(j < d ? j : d - 1) * nq4;
#pragma unroll
            for (int s = 0; s < NS; ++s) dst[s] = M4[base + qc[s]];
        };
        float4 ring[R][NS];
#pragma unroll
        for (int u = 0; u + 1 < R || u == 0; ++u) loadrow(jfirst + 16 * u, ring[u]);
        for (int j0 = jfirst; j0 < d + 16 * R; j0 += 16 * R) {  // uniform trip count over the workgroup
#pragma unroll
            for (int u = 0; u < R; ++u) {
                const int j = j0 + 16 * u;
                if constexpr (R > 1) {
                    loadrow(j + 16 * (R - 1), ring[(u + R - 1) % R]);
                    __builtin_amdgcn_sched_barrier(0);
                }
                float p[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int s = 0; s < NS; ++s) {
                    const float4 m = ring[u][s];
#pragma unroll
                    for (int r = 0; r < 4; ++r)
                        p[r] = fmaf(q[s][r].x, m.x, fmaf(q[s][r].y, m.y, fmaf(q[s][r].z, m.z, fmaf(q[s][r].w, m.w, p[r]))));
                }
                if constexpr (R == 1) loadrow(j + 16, ring[0]);
#pragma unroll
                for (int r = 0; r < 4; ++r) p[r] = row16_sum(p[r]);
                if (li < 4 && j < d) {
                    const float v = li == 0 ? p[0] : (li == 1 ? p[1] : (li == 2 ? p[2] : p[3]));
                    sY[li * d + j] = c0 == 0 ? v : sY[li * d + j] + v;  // same lane owns (li, j) in every pass
                }
            }
        }
    }
    __syncthreads();
    for (int f = tid; f < rows * nq4; f += 256) {
        const int r = f / nq4, c = f % nq4;
        const float4 y = *reinterpret_cast<const float4 *>(&sY[r * d + 4 * c]);
        const int64_t o = (int64_t)s_b[r] * d + 4 * c;
        *reinterpret_cast<float4 *>(a.occ_h + o) = y;
        if (a.occ_t) *reinterpret_cast<float4 *>(a.occ_t + o) = make_float4(-y.x, -y.y, -y.z, -y.w);
        if (derived && a.src.occ_v) {  // RESCAL: the tail's occurrence row g * (E[h] Proj[r])
            const float gr = r == 0 ? qg[0] : (r == 1 ? qg[1] : (r == 2 ? qg[2] : qg[3]));
            *reinterpret_cast<float4 *>(a.src.occ_v + o) = scaled4(gr, *reinterpret_cast<const float4 *>(a.src.resid + o));
        }
    }
}

static size_t thin_dx_lds_bytes(int d) { return sizeof(float) * 4 * (size_t)d; }

// One sweep of a tile: acc (+)= X[32 x d] * B over all supersteps for this wave's columns
// [n0, n0 + wcols).  Everything inside the loop is free of branches: addresses are clamped
// into the projection instead of predicating the loads (the staged X is zero for k >= d, and a
// lane beyond wcols computes columns nobody stores), the prefetch of a superstep past the end
// re-reads the last one, and the superstep count is rounded up to whole ring turns with the X
// operand selected to zero.  A branch around a load makes the compiler wait for every load
// in flight at each step, which turns the prefetch ring into a depth of one.
//   MODE 0/1: B[k][j] = M[k][n0 + 4 li + e], one float4 per k row per lane;
//   MODE 2:   B[k][j] = M[n0 + 16 e + li][k], a lane's float4 along k serves the four steps.
template <int MODE>
struct BLoader {
    const float *base[4];
    int d, nq, kk;
    __device__ __forceinline__ void init(const float *M, int d_, int nq_, int n0, int wcols, int li, int kk_)
    {
        d = d_, nq = nq_, kk = kk_;
        if constexpr (MODE != 2) {
            const int col = n0 + (4 * li < wcols ? 4 * li : 0);
#pragma unroll
            for (int s = 0; s < 4; ++s) base[s] = M + col;
        } else {
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const int col = 16 * e + li;
                base[e] = M + (int64_t)(n0 + (col < wcols ? col : 0)) * d;
            }
        }
    }
    __device__ __forceinline__ void load(int q, float4 *dst) const
    {
        q = q < nq ? q : nq - 1;
        if constexpr (MODE != 2) {
#pragma unroll
            for (int s = 0; s < 4; ++s) {
                const int k = 16 * q + 4 * kk + s;
                dst[s] = *reinterpret_cast<const float4 *>(base[s] + (int64_t)(k < d ? k : d - 1) * d);
            }
        } else {
            const int k = 16 * q + 4 * kk;
#pragma unroll
            for (int e = 0; e < 4; ++e) dst[e] = *reinterpret_cast<const float4 *>(base[e] + (k < d ? k : d - 4));
        }
    }
};

// Ring of kRing slots: step qq consumes slot qq % kRing and first refills the slot consumed one
// step earlier with superstep qq + kRing - 1, so kRing - 1 supersteps are always in flight and
// the loads are issued ahead of the matrix-core work of the step (pinned by the scheduling
// barrier; left alone the compiler sinks them below it and the ring degenerates to depth 1).
// ring_prime() issues the first kRing - 1 supersteps; a tile calls it before it stages its left
// operand (the projection only depends on the tile's relation), so those loads fly during the
// index chain and the row gathers of the staging.
template <int MODE, int RING>
__device__ __forceinline__ void ring_prime(const BLoader<MODE> &bl, float4 (&ring)[RING][4])
{
#pragma unroll
    for (int u = 0; u + 1 < RING; ++u) bl.load(u, ring[u]);
}

template <int MODE, bool TWO, int RING>
__device__ __forceinline__ void gemm_sweep(const BLoader<MODE> &bl, float4 (&ring)[RING][4], const float *sX, int pitch,
                                           int li, int kk, floatx4 (&acc_lo)[4], floatx4 (&acc_hi)[4])
{
    const int nq = bl.nq;
    const float *xlo = sX + li * pitch + 4 * kk, *xhi = sX + (16 + li) * pitch + 4 * kk;
    for (int q = 0; q < nq; q += RING) {
#pragma unroll
        for (int u = 0; u < RING; ++u) {
            const int qq = q + u;
            bl.load(qq + RING - 1, ring[(u + RING - 1) % RING]);
            __builtin_amdgcn_sched_barrier(0);
            float4 bc[4];
#pragma unroll
            for (int s = 0; s < 4; ++s) bc[s] = ring[u][s];
            const bool live = qq < nq;
            const int qc = live ? qq : nq - 1;
            float4 alo = *reinterpret_cast<const float4 *>(xlo + 16 * qc);
            float4 ahi = TWO ? *reinterpret_cast<const float4 *>(xhi + 16 * qc) : make_float4(0.f, 0.f, 0.f, 0.f);
            if (!live) alo = make_float4(0.f, 0.f, 0.f, 0.f), ahi = alo;
            const float al[4] = {alo.x, alo.y, alo.z, alo.w}, ah[4] = {ahi.x, ahi.y, ahi.z, ahi.w};
            if constexpr (MODE != 2) {
#pragma unroll
                for (int s = 0; s < 4; ++s) {
                    const float bv[4] = {bc[s].x, bc[s].y, bc[s].z, bc[s].w};
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        acc_lo[e] = __builtin_amdgcn_mfma_f32_16x16x4f32(al[s], bv[e], acc_lo[e], 0, 0, 0);
                        if constexpr (TWO)
                            acc_hi[e] = __builtin_amdgcn_mfma_f32_16x16x4f32(ah[s], bv[e], acc_hi[e], 0, 0, 0);
                    }
                }
            } else {
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const float bv[4] = {bc[e].x, bc[e].y, bc[e].z, bc[e].w};
#pragma unroll
                    for (int s = 0; s < 4; ++s) {
                        acc_lo[e] = __builtin_amdgcn_mfma_f32_16x16x4f32(al[s], bv[s], acc_lo[e], 0, 0, 0);
                        if constexpr (TWO)
                            acc_hi[e] = __builtin_amdgcn_mfma_f32_16x16x4f32(ah[s], bv[s], acc_hi[e], 0, 0, 0);
                    }
                }
            }
        }
    }
}

// MODE 0: forward TransR   x = E[h]-E[t], y = x M + R[r], score = ||y||_p
// MODE 1: forward RESCAL   x = E[h],      y = x M,        score = y . E[t]
// MODE 2: backward dX      x = xs rows,   y = x M^T -> occ_h = y, occ_t = -y (when occ_t is set)
// MODE 3: list rows        x = E[h]-E[t] (t = -1: no row), y = x M + rs R[r] -> resid rows in list order;
//         h, t, rs are indexed by the sorted position itself (no perm), no score
template <int MODE, int RING = kRing>
__device__ __forceinline__ void transr_gemm_body(const GemmArgs &a, float *lds, int bid)
{
    // Workgroups [0, max_tiles) take the planned 32-triple tiles, the following `thin_groups`
    // stream the thin group tails.  The tiles come first because each is one long chain of
    // dependent loads and matrix-core steps (about 20 us whatever else runs); the thin
    // workgroups then fill the remaining slots and the memory bandwidth.
    if (bid >= a.max_tiles) {
        if constexpr (MODE == 2) {
            const int ns = (a.d / 4 + 15) / 16;  // k-quads per lane of a 16-lane row group
            if (ns <= 1) transr_thin_dx_body<1>(a, lds, bid - a.max_tiles);
            else if (ns <= 2) transr_thin_dx_body<2>(a, lds, bid - a.max_tiles);
            else transr_thin_dx_body<4>(a, lds, bid - a.max_tiles);
        } else {
            transr_thin_fwd_body<MODE>(a, lds, bid - a.max_tiles);
        }
        return;
    }
    const int tile = bid;
    if (tile >= a.plan.num_tiles[0]) return;
    const int d = a.d;
    const int kpad = (d + 15) & ~15;
    const int pitch = kpad + 4;
    float *sX = lds;                 // [kTM][pitch]
    float *sRed = lds + kTM * pitch; // [4][kTM]
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    // everything the tile needs to know comes from the plan in one round trip
    const int p0 = a.plan.tile_p0[tile], seg_end = a.plan.tile_end[tile];
    const int64_t rid = a.plan.tile_rid[tile];
    const int rows = seg_end - p0 < kTM ? seg_end - p0 : kTM;
    if (rows <= kThin) return;  // streamed by a thin workgroup
    const float *M = a.proj + rid * (int64_t)d * d;
    const int li = lane & 15, kk = lane >> 4;

    // The projection's first supersteps are requested before the left operand is staged: they
    // depend on the relation only and fly during the index chain and the row gathers below.
    auto wave_cols = [&](int c0, int &n0, int &wcols) {  // 256 output columns per sweep, split over the waves
        const int span = d - c0 < 256 ? d - c0 : 256;
        const int cw = ((span / 4 + 3) / 4) * 4;  // columns per wave, a multiple of 4
        n0 = c0 + wave * cw;
        wcols = n0 >= c0 + span ? 0 : (c0 + span - n0 < cw ? c0 + span - n0 : cw);
    };
    BLoader<MODE> bl;
    float4 ring[RING][4];
    {
        int n0, wcols;
        wave_cols(0, n0, wcols);
        if (wcols > 0) {  // per wave; a wave without columns (narrow rows) sits the sweep out
            bl.init(M, d, kpad / 16, n0, wcols, li, kk);
            ring_prime<MODE, RING>(bl, ring);
        }
        __builtin_amdgcn_sched_barrier(0);
    }

    // triple ids of the tile first (one dependent-load chain per row instead of one per element)
    __shared__ int s_b[kTM];
    __shared__ int64_t s_h[kTM], s_t[kTM];
    __shared__ float s_rs[MODE == 3 ? kTM : 1];
    __shared__ float s_coef[MODE == 2 ? kTM : 1], s_g[MODE == 2 ? kTM : 1];
    __shared__ int64_t s_qoff[MODE == 2 ? kTM : 1];
    const bool derived = MODE == 2 && a.xs == nullptr;  // the upstream rows are formed while staging (BwdSrc)
    if (tid < kTM) {
        int b;
        if constexpr (MODE == 3) b = p0 + (tid < rows ? tid : 0);
        else if (derived) {
            const RowMeta m = bwd_row_meta(a.src, p0 + (tid < rows ? tid : 0), d);
            b = m.b;
            if constexpr (MODE == 2) s_coef[tid] = m.coef, s_qoff[tid] = m.qoff, s_g[tid] = a.src.dpos ? a.src.dpos[m.b] : 0.0f;
        } else b = tid < rows ? (a.perm ? a.perm[p0 + tid] : p0 + tid) : 0;
        s_b[tid] = b;
        if constexpr (MODE != 2) {
            s_h[tid] = a.h[b];
            s_t[tid] = a.t[b];
        }
        if constexpr (MODE == 3) s_rs[tid] = a.rs[b];
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
                        if (derived) {  // uniform
                            v[q] = *reinterpret_cast<const float4 *>(bwd_qbase(a.src) + s_qoff[row] + k4);
                            if (a.src.occ_v) u[q] = *reinterpret_cast<const float4 *>(a.src.resid + (int64_t)s_b[row] * d + k4);
                        } else {
                            v[q] = *reinterpret_cast<const float4 *>(a.xs + (int64_t)(p0 + row) * d + k4);
                        }
                    } else {
                        if (MODE == 1 && a.xs)  // uniform: left operand rows given in sorted order
                            v[q] = *reinterpret_cast<const float4 *>(a.xs + (int64_t)(p0 + row) * d + k4);
                        else
                            v[q] = *reinterpret_cast<const float4 *>(a.ent + s_h[row] * (int64_t)d + k4);
                        if constexpr (MODE == 0)
                            u[q] = *reinterpret_cast<const float4 *>(a.ent + s_t[row] * (int64_t)d + k4);
                        if constexpr (MODE == 3) {
                            if (s_t[row] >= 0) u[q] = *reinterpret_cast<const float4 *>(a.ent + s_t[row] * (int64_t)d + k4);
                        }
                    }
                }
            }
#pragma unroll
            for (int q = 0; q < kStageBatch; ++q) {
                const int f = f0 + 256 * q;
                if (f < kTM * per_row) {
                    const int row = f / per_row, k4 = (f % per_row) * 4;
                    float4 x = make_float4(v[q].x - u[q].x, v[q].y - u[q].y, v[q].z - u[q].z, v[q].w - u[q].w);
                    if constexpr (MODE == 2) {
                        if (derived) {
                            const bool l1 = !a.src.rescal && a.src.norm_p == 1;
                            x = row < rows ? scaled4(s_coef[row], l1 ? sgn4(v[q]) : v[q]) : make_float4(0.f, 0.f, 0.f, 0.f);
                            if (a.src.occ_v && row < rows && k4 < d)  // RESCAL: the tail's occurrence row g * (E[h] Proj[r])
                                *reinterpret_cast<float4 *>(a.src.occ_v + (int64_t)s_b[row] * d + k4) = scaled4(s_g[row], u[q]);
                        }
                    }
                    *reinterpret_cast<float4 *>(&sX[row * pitch + k4]) = x;
                }
            }
        }
    }
    __syncthreads();

    const bool two_blocks = rows > 16;
    float rowsum[8];  // norm / dot partials for rows 4*kk + r (+16)
#pragma unroll
    for (int r = 0; r < 8; ++r) rowsum[r] = 0.0f;

    for (int c0 = 0; c0 < d; c0 += 256) {
        int n0, wcols;
        wave_cols(c0, n0, wcols);
        floatx4 acc_lo[4], acc_hi[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) acc_lo[e] = floatx4{0.f, 0.f, 0.f, 0.f}, acc_hi[e] = floatx4{0.f, 0.f, 0.f, 0.f};
        if (c0 > 0 && wcols > 0) {  // (the first sweep's ring was primed before the staging)
            bl.init(M, d, kpad / 16, n0, wcols, li, kk);
            ring_prime<MODE, RING>(bl, ring);
        }
        // epilogue operands that do not depend on the products: the relation row (TransR) is requested
        // ahead of the sweep, the tail rows of this lane's eight triples (RESCAL) in one batch behind it
        const int ecol = 4 * li < wcols ? n0 + 4 * li : 0;
        float4 erow[MODE == 1 ? 8 : 1];
        if constexpr (MODE == 0 || MODE == 3) erow[0] = *reinterpret_cast<const float4 *>(a.rel + rid * (int64_t)d + ecol);

        if (wcols > 0) {
            if (two_blocks) gemm_sweep<MODE, true, RING>(bl, ring, sX, pitch, li, kk, acc_lo, acc_hi);
            else gemm_sweep<MODE, false, RING>(bl, ring, sX, pitch, li, kk, acc_lo, acc_hi);
        }
        if constexpr (MODE == 1) {  // one batch of unconditional loads (eight rows would not fit beside the ring)
#pragma unroll
            for (int q = 0; q < 8; ++q) {
                const int row = 16 * (q >> 2) + 4 * kk + (q & 3);
                erow[q] = *reinterpret_cast<const float4 *>(a.ent + s_t[row < rows ? row : 0] * (int64_t)d + ecol);
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
                        if constexpr (MODE == 3) {
                            const float4 rv = erow[0];
                            const float f = s_rs[row];  // +-1 or 0: exact products
                            y[0] += f * rv.x, y[1] += f * rv.y, y[2] += f * rv.z, y[3] += f * rv.w;
                        } else if constexpr (MODE == 0) {
                            const float4 rv = erow[0];
                            y[0] += rv.x, y[1] += rv.y, y[2] += rv.z, y[3] += rv.w;
                            float s = 0.0f;
#pragma unroll
                            for (int e = 0; e < 4; ++e) s += a.norm_p == 1 ? fabsf(y[e]) : y[e] * y[e];
                            rowsum[4 * blk + r] += s;
                        } else {
                            const float4 tv = erow[MODE == 1 ? 4 * blk + r : 0];
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

template <int MODE>
__global__ __launch_bounds__(256, KGE_TR_OCC) void transr_gemm_kernel(GemmArgs a, FusedInsp fi)
{
    extern __shared__ __align__(16) float lds[];
    if (fused_insp_block(fi, reinterpret_cast<uint32_t *>(lds))) return;  // an inspector workgroup riding along
    transr_gemm_body<MODE>(a, lds, (int)blockIdx.x - fi.blocks);
}

// ---- forward TransR with the back rows (GemmArgs::back) ---------------------------------------------------
// The entity gradients of the backward pass are coef_b * (phi(y_b) Proj^T): everything but the coefficient is known
// at the end of the forward tile.
//
// A thin group (at most kThin triples, most distinct relations of a long-tailed batch and four fifths of the
// projection bytes) reads its projection ONCE for both products: the workgroup requests all of it at the start
// (RMAX * NQ 128-bit loads per thread, the whole 4 d^2 bytes in flight) and keeps it in registers.  Thread
// (row group rg = lane / 16 + 4 wave, li = lane % 16) holds rows j = rg + 16 i and the quads c = li + 16 s of each.
//   y[b][c] = sum_j x[b][j] M[j][c]: per-thread sums over its rows, the four row groups of a wave added with two
//             cross-lane steps, the four waves through LDS in a fixed order;
//   z[b][j] = sum_c phi(y)[b][c] M[j][c]: per-thread dot products, the sixteen lanes of a row added with four
//             DPP steps (as the thin dX pass does).
// Needs RMAX * NQ * 4 registers for the projection: row widths up to 208 (NQ = ceil(d / 64), RMAX rows per thread).
template <int NQ>
__device__ __forceinline__ void transr_thin_both_body(const GemmArgs &a, float *lds, int g)
{
    constexpr int RMAX = NQ == 1 ? 4 : (NQ == 2 ? 8 : (NQ == 3 ? 12 : 13));
    constexpr int RX = 16 * RMAX;  // >= d
    const ThinTile tt = thin_tile_of_group(a.num_unique, a.seg_offsets, g);
    const int rows = tt.rows;
    if (rows == 0) return;
    const int d = a.d, nq4 = d >> 2, tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int li = lane & 15, sub = lane >> 4, rg = 4 * wave + sub;
    float *sx = lds;                                        // [4][RX] x rows, zero beyond d and beyond `rows`
    float4 *sW = reinterpret_cast<float4 *>(lds + 4 * RX);  // [4 waves][4 rows][64 quads]
    float4 *sq = sW + 4 * 4 * 64;                           // [4 rows][64 quads] phi(y), zero beyond the row
    float *sz = reinterpret_cast<float *>(sq + 4 * 64);     // [4][RX]
    __shared__ int s_b[kThin];
    __shared__ int64_t s_h[kThin], s_t[kThin];
    const int64_t rid = a.unique_ids[g];
    const float4 *M4 = reinterpret_cast<const float4 *>(a.proj + rid * (int64_t)d * d);
    float4 m[RMAX][NQ];
#pragma unroll
    for (int i = 0; i < RMAX; ++i) {
        const int j = rg + 16 * i;
        const int64_t base = (int64_t)(j < d ? j : d - 1) * nq4;  // clamped: unconditional loads, x is zero there
#pragma unroll
        for (int q = 0; q < NQ; ++q) {
            const int c = li + 16 * q;
            m[i][q] = M4[base + (c < nq4 ? c : 0)];
        }
    }
    __builtin_amdgcn_sched_barrier(0);
    if (tid < kThin) {
        const int b = tid < rows ? a.perm[tt.p0 + tid] : 0;
        s_b[tid] = b;
        s_h[tid] = a.h[b];
        s_t[tid] = a.t[b];
    }
    for (int k = tid; k < 4 * RX; k += 256) sx[k] = 0.0f;
    __syncthreads();
    for (int f = tid; f < rows * nq4; f += 256) {
        const int r = f / nq4, k4 = (f % nq4) * 4;
        const float4 v = *reinterpret_cast<const float4 *>(a.ent + s_h[r] * (int64_t)d + k4);
        const float4 u = *reinterpret_cast<const float4 *>(a.ent + s_t[r] * (int64_t)d + k4);
        *reinterpret_cast<float4 *>(&sx[r * RX + k4]) = make_float4(v.x - u.x, v.y - u.y, v.z - u.z, v.w - u.w);
    }
    __syncthreads();
    // y = x M: this thread's rows, then the wave's four row groups
#pragma unroll
    for (int b = 0; b < 4; ++b) {
        float4 acc[NQ];
#pragma unroll
        for (int q = 0; q < NQ; ++q) acc[q] = make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
        for (int i = 0; i < RMAX; ++i) {
            const float xv = sx[b * RX + rg + 16 * i];
#pragma unroll
            for (int q = 0; q < NQ; ++q) {
                acc[q].x = fmaf(xv, m[i][q].x, acc[q].x);
                acc[q].y = fmaf(xv, m[i][q].y, acc[q].y);
                acc[q].z = fmaf(xv, m[i][q].z, acc[q].z);
                acc[q].w = fmaf(xv, m[i][q].w, acc[q].w);
            }
        }
#pragma unroll
        for (int q = 0; q < NQ; ++q) {
            float v[4] = {acc[q].x, acc[q].y, acc[q].z, acc[q].w};
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                v[e] += __shfl_xor(v[e], 16, kWave);
                v[e] += __shfl_xor(v[e], 32, kWave);
            }
            if (sub == 0) sW[(wave * 4 + b) * 64 + li + 16 * q] = make_float4(v[0], v[1], v[2], v[3]);
        }
    }
    __syncthreads();
    {   // thread (row b = wave, quad c = lane): the four waves' sums in order, the relation row, the score
        const int b = wave, c = lane;
        float4 y = sW[b * 64 + c];
#pragma unroll
        for (int w = 1; w < 4; ++w) {
            const float4 v = sW[(w * 4 + b) * 64 + c];
            y.x += v.x, y.y += v.y, y.z += v.z, y.w += v.w;
        }
        float sum = 0.0f;
        float4 q = make_float4(0.f, 0.f, 0.f, 0.f);
        if (c < nq4 && b < rows) {
            const float4 rv = *reinterpret_cast<const float4 *>(a.rel + rid * (int64_t)d + 4 * c);
            y.x += rv.x, y.y += rv.y, y.z += rv.z, y.w += rv.w;
            sum = a.norm_p == 1 ? fabsf(y.x) + fabsf(y.y) + fabsf(y.z) + fabsf(y.w)
                                : y.x * y.x + y.y * y.y + y.z * y.z + y.w * y.w;
            if (a.resid) *reinterpret_cast<float4 *>(a.resid + (int64_t)s_b[b] * d + 4 * c) = y;
            q = a.norm_p == 1 ? sgn4(y) : y;
        }
        sq[b * 64 + c] = q;
        sum = wave_sum(sum);
        if (lane == 0 && b < rows && a.pos) a.pos[s_b[b]] = a.norm_p == 2 ? sqrtf(sum) : sum;
    }
    __syncthreads();
    // z = phi(y) M^T
#pragma unroll
    for (int b = 0; b < 4; ++b) {
        float4 qv[NQ];
#pragma unroll
        for (int q = 0; q < NQ; ++q) qv[q] = sq[b * 64 + li + 16 * q];  // zero beyond the row: clamped quads add nothing
#pragma unroll
        for (int i = 0; i < RMAX; ++i) {
            float p = 0.0f;
#pragma unroll
            for (int q = 0; q < NQ; ++q)
                p = fmaf(qv[q].x, m[i][q].x, fmaf(qv[q].y, m[i][q].y, fmaf(qv[q].z, m[i][q].z, fmaf(qv[q].w, m[i][q].w, p))));
            p = row16_sum(p);
            if (li == 0) sz[b * RX + rg + 16 * i] = p;
        }
    }
    __syncthreads();
    for (int f = tid; f < rows * nq4; f += 256) {
        const int r = f / nq4, k4 = (f % nq4) * 4;
        *reinterpret_cast<float4 *>(a.back + (int64_t)s_b[r] * d + k4) = *reinterpret_cast<const float4 *>(&sz[r * RX + k4]);
    }
}

constexpr int kThinBothMaxDim = 208;
constexpr int kBackRing = kRing;  // prefetch stages of the tiles in this kernel (4 to 8 stages, which its register budget would allow, measured slower)
static size_t thin_both_lds_bytes(int d)
{
    if (d > kThinBothMaxDim) return 0;
    const int nq = (d / 4 + 15) / 16, rmax = nq == 1 ? 4 : (nq == 2 ? 8 : (nq == 3 ? 12 : 13));
    return sizeof(float) * (size_t)(8 * 16 * rmax) + sizeof(float4) * (size_t)(4 * 4 * 64 + 4 * 64);
}

// Tiles: the second sweep (the dX body on the rows this workgroup has just written, coefficient 1) follows the
// first at once: no launch, no index chains, no ramp or tail between them; the barrier makes the rows visible to
// all waves of the workgroup.  Two workgroups per CU: the thin groups' projections live in registers.
__global__ __launch_bounds__(256, 2) void transr_fwd_back_kernel(GemmArgs a, FusedInsp fi)
{
    extern __shared__ __align__(16) float lds[];
    if (fused_insp_block(fi, reinterpret_cast<uint32_t *>(lds))) return;
    const int bid = (int)blockIdx.x - fi.blocks;
    if (bid >= a.max_tiles && a.d <= kThinBothMaxDim) {
        const int nq = (a.d / 4 + 15) / 16;
        if (nq <= 1) transr_thin_both_body<1>(a, lds, bid - a.max_tiles);
        else if (nq == 2) transr_thin_both_body<2>(a, lds, bid - a.max_tiles);
        else if (nq == 3) transr_thin_both_body<3>(a, lds, bid - a.max_tiles);
        else transr_thin_both_body<4>(a, lds, bid - a.max_tiles);
        return;
    }
    transr_gemm_body<0, kBackRing>(a, lds, bid);
    __syncthreads();
    GemmArgs z = a;
    z.xs = nullptr, z.pos = nullptr, z.resid = nullptr, z.occ_h = a.back, z.occ_t = nullptr;
    z.src = BwdSrc{a.ent, a.resid, nullptr, nullptr, a.h, a.t, a.perm, a.norm_p, 0, nullptr, 1};
    transr_gemm_body<2, kBackRing>(z, lds, bid);
}

static size_t gemm_lds_bytes(int d)  // the larger of the tile layout and the thin layouts
{
    const int kpad = (d + 15) & ~15;
    const size_t tile = sizeof(float) * ((size_t)kTM * (kpad + 4) + 4 * kTM);
    const size_t thin = thin_fwd_lds_bytes(d) > thin_dx_lds_bytes(d) ? thin_fwd_lds_bytes(d) : thin_dx_lds_bytes(d);
    return tile > thin ? tile : thin;
}

static int thin_groups(const kge_tables *tab, const kge_batch *bat)
{
    return (int)(bat->batch < tab->n_rel ? bat->batch : tab->n_rel);
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

bool transr_grouped_path_ok(const kge_tables *tab, const kge_batch *bat)
{
    return mfma_path_ok(tab, bat) && gemm_lds_bytes((int)tab->dim) <= kMaxGemmLds;
}

// ---- backward kernels ----------------------------------------------------------------------
#ifndef KGE_TR_DM_CHUNK
#define KGE_TR_DM_CHUNK 256
#endif
constexpr int kDmChunk = KGE_TR_DM_CHUNK;  // triples of one relation group per dM work item (at most 256: one per thread when staging)
constexpr int kDmXP = 36;      // LDS pitch of a staged left-operand row (32 columns + 4: the four lane groups of an MFMA step read distinct banks)

struct DmArgs {
    const float *xs, *qs;  // operand rows in sorted order [B, d]; null: formed from `src` (BwdSrc)
    const int32_t *seg_offsets;
    TilePlan plan;   // tiles of kDmChunk positions, with split bookkeeping
    float *dm;       // [U, d, d]
    float *part;     // [max_slots, d, d] partial results of split groups
    int d;
    const int32_t *num_unique;
    BwdSrc src;
    // Factored output (kge_grads.aux_x / aux_q): a group of at most factor_max (<= kThin) triples writes its
    // operand rows x_p, q_p to fx[p], fq[p] (p = its sorted positions) instead of the dense d x d sum of
    // their outer products.  fx null: every group dense.
    float *fx, *fq;
    int factor_max;
};

// dM of a group of at most kThin triples: four outer products written as one contiguous stream.
// Thread (phase, cq) keeps its column quad of the Q rows in registers and walks the rows
// k = phase, phase + P, ... of the output, so consecutive threads write consecutive 16 bytes.
// With factored output the rows themselves are the result (2 * rows * d floats instead of d * d).
__device__ __forceinline__ void transr_thin_dm_body(const DmArgs &a, float *lds, int g)
{
    if (g >= a.num_unique[0]) return;
    const int s0 = a.seg_offsets[g], rows = a.seg_offsets[g + 1] - s0;
    if (rows > kThin) return;
    const int d = a.d, nq4 = d >> 2, tid = threadIdx.x;
    const int P = 256 / nq4;
    const bool derived = a.xs == nullptr;
    // (the same addresses in every lane: scalar loads)
    const float *xh[4], *xt[4], *qrow[4];
    float qcoef[4];
#pragma unroll
    for (int r = 0; r < 4; ++r) {
        const int p = s0 + (r < rows ? r : 0);
        if (derived) {
            const RowMeta m = bwd_row_meta(a.src, p, d);
            xh[r] = a.src.ent + m.xh * d, xt[r] = a.src.ent + m.xt * d;
            qrow[r] = bwd_qbase(a.src) + m.qoff, qcoef[r] = m.coef;
        } else {
            xh[r] = a.xs + (int64_t)p * d, xt[r] = xh[r], qrow[r] = a.qs + (int64_t)p * d, qcoef[r] = 1.0f;
        }
    }
    const bool sub_t = derived && !a.src.rescal, sign_rows = derived && !a.src.rescal && a.src.norm_p == 1;
    const bool factored = a.fx && rows <= a.factor_max;
    float4 *sXT = reinterpret_cast<float4 *>(lds);  // [d] x[0..3][k]
    for (int f = tid; f < 4 * nq4; f += 256) {
        const int r = f / nq4, k4 = (f % nq4) * 4;
        const float *ph = r == 0 ? xh[0] : (r == 1 ? xh[1] : (r == 2 ? xh[2] : xh[3]));
        const float *pt = r == 0 ? xt[0] : (r == 1 ? xt[1] : (r == 2 ? xt[2] : xt[3]));
        float4 v = *reinterpret_cast<const float4 *>(ph + k4);
        const float4 u = *reinterpret_cast<const float4 *>(pt + k4);
        if (sub_t) v = make_float4(v.x - u.x, v.y - u.y, v.z - u.z, v.w - u.w);
        if (r >= rows) v = make_float4(0.f, 0.f, 0.f, 0.f);
        if (factored) {
            if (r < rows) *reinterpret_cast<float4 *>(a.fx + (int64_t)(s0 + r) * d + k4) = v;
        } else {
            float *col = reinterpret_cast<float *>(sXT + k4) + r;
            col[0] = v.x, col[4] = v.y, col[8] = v.z, col[12] = v.w;
        }
    }
    const int cq = tid % nq4, ph = tid / nq4;
    float4 q[4];
#pragma unroll
    for (int r = 0; r < 4; ++r) {
        q[r] = *reinterpret_cast<const float4 *>(qrow[r] + 4 * cq);
        if (derived) q[r] = scaled4(qcoef[r], sign_rows ? sgn4(q[r]) : q[r]);
        if (r >= rows) q[r] = make_float4(0.f, 0.f, 0.f, 0.f);
    }
    if (factored) {
        if (ph == 0) {
#pragma unroll
            for (int r = 0; r < 4; ++r)
                if (r < rows) *reinterpret_cast<float4 *>(a.fq + (int64_t)(s0 + r) * d + 4 * cq) = q[r];
        }
        return;
    }
    __syncthreads();
    if (ph >= P) return;
    float4 *out = reinterpret_cast<float4 *>(a.dm + (int64_t)g * d * d);
    for (int k = ph; k < d; k += P) {
        const float4 x = sXT[k];
        float4 o;
        o.x = fmaf(x.w, q[3].x, fmaf(x.z, q[2].x, fmaf(x.y, q[1].x, x.x * q[0].x)));
        o.y = fmaf(x.w, q[3].y, fmaf(x.z, q[2].y, fmaf(x.y, q[1].y, x.x * q[0].y)));
        o.z = fmaf(x.w, q[3].z, fmaf(x.z, q[2].z, fmaf(x.y, q[1].z, x.x * q[0].z)));
        o.w = fmaf(x.w, q[3].w, fmaf(x.z, q[2].w, fmaf(x.y, q[1].w, x.x * q[0].w)));
        out[(int64_t)k * nq4 + cq] = o;
    }
}

// K loop of a dM work item: acc (+)= X[p, i0 .. i0+31]^T Q[p, n0 .. n0+wcols) over the item's n
// positions.  The left operand comes from LDS (sX: [16 * nq][kDmXP], staged by transr_dm_body with
// zeros beyond n and beyond the row width), the right operand straight from memory through the row
// offsets sOff (one 128-bit load per position and lane).  As in gemm_sweep the loads of a superstep
// are free of branches: a position past the end re-reads the last one (its X is zero), a lane
// outside the column range reads column n0 and produces values nobody stores, and the issue order of
// the prefetch is pinned.  SIGN: the right operand is sign(row) (TransR, L1: the coefficient sits in X).
template <bool TWO, bool SIGN>
__device__ __forceinline__ void dm_sweep(const float *qbase, const float *sX, const int64_t *sOff, int n, int nq, int n0,
                                         int wcols, int li, int kk, floatx4 (&acc_lo)[4], floatx4 (&acc_hi)[4])
{
    const float *qb = qbase + n0 + (4 * li < wcols ? 4 * li : 0);
    auto load_stage = [&](int q, float4 (&bv)[4]) {
#pragma unroll
        for (int s = 0; s < 4; ++s) {
            const int i = 16 * q + 4 * kk + s;
            bv[s] = *reinterpret_cast<const float4 *>(qb + sOff[i < n ? i : n - 1]);
        }
    };
    // Most work items are short (a group of 5..16 triples is a single superstep), so unlike in
    // gemm_sweep the prefetch is skipped past the end: a uniform branch per superstep, none per load.
    float4 ring[kDmRing][4];
#pragma unroll
    for (int u = 0; u + 1 < kDmRing; ++u)
        if (u < nq) load_stage(u, ring[u]);
    for (int q = 0; q < nq; q += kDmRing) {
#pragma unroll
        for (int u = 0; u < kDmRing; ++u) {
            const int qq = q + u;
            if (qq >= nq) break;
            if (qq + kDmRing - 1 < nq) load_stage(qq + kDmRing - 1, ring[(u + kDmRing - 1) % kDmRing]);
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int s = 0; s < 4; ++s) {
                const int i = 16 * qq + 4 * kk + s;
                const float al = sX[i * kDmXP + li];
                const float ah = TWO ? sX[i * kDmXP + 16 + li] : 0.0f;
                const float4 bq = SIGN ? sgn4(ring[u][s]) : ring[u][s];
                const float b4[4] = {bq.x, bq.y, bq.z, bq.w};
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    acc_lo[e] = __builtin_amdgcn_mfma_f32_16x16x4f32(al, b4[e], acc_lo[e], 0, 0, 0);
                    if constexpr (TWO) acc_hi[e] = __builtin_amdgcn_mfma_f32_16x16x4f32(ah, b4[e], acc_hi[e], 0, 0, 0);
                }
            }
        }
    }
}

// dM of a group of kThin + 1 .. kDmSmall triples (most of the groups that are not thin), by ONE workgroup:
// the group's x rows are staged whole in LDS (coefficients folded in), each wave loads its columns of the
// q rows once into registers, and the row blocks of the d x d result follow one another with no further
// loads.  As (chunk, row block) work items such a group costs ceil(d / 32) workgroups that each walk the
// same index chain and re-read the same q rows for a single superstep of matrix-core work.
constexpr int kDmSmall = 32;
constexpr int kDmSmallLdsFloats = 256 * kDmXP;  // what the small-group layout may take (36 KB: three workgroups per CU with room to spare)
__host__ __device__ inline bool dm_small_fits(int d) { return kDmSmall * (d + 4) <= kDmSmallLdsFloats; }

template <bool SIGN>
__device__ __forceinline__ void transr_dm_small_body(const DmArgs &a, float *lds, int s0, int n, float *dst)
{
    const int d = a.d, pitch = d + 4, nq4 = d >> 2;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, li = lane & 15, kk = lane >> 4;
    const int nq = (n + 15) / 16;  // 1 or 2
    const bool derived = a.xs == nullptr;
    float *sX = lds;                                                      // [kDmSmall][pitch]
    int64_t *sOff = reinterpret_cast<int64_t *>(lds + kDmSmallLdsFloats);  // [kDmSmall]
    __shared__ int64_t s_xh[kDmSmall], s_xt[kDmSmall];
    __shared__ float s_c[kDmSmall];
    if (tid < kDmSmall) {
        const int p = s0 + (tid < n ? tid : n - 1);
        if (derived) {
            const RowMeta m = bwd_row_meta(a.src, p, d);
            s_xh[tid] = m.xh * d, s_xt[tid] = m.xt * d, s_c[tid] = m.coef, sOff[tid] = m.qoff;
        } else {
            s_xh[tid] = (int64_t)p * d, s_xt[tid] = s_xh[tid], s_c[tid] = 1.0f, sOff[tid] = (int64_t)p * d;
        }
    }
    __syncthreads();
    const float *xbase = derived ? a.src.ent : a.xs;
    const bool sub_t = derived && !a.src.rescal;
    {
        constexpr int kBatch = 4;
        const int total = 16 * nq * nq4;
        for (int f0 = tid; f0 < total; f0 += 256 * kBatch) {
            float4 v[kBatch], u[kBatch];
#pragma unroll
            for (int q = 0; q < kBatch; ++q) {
                const int f = f0 + 256 * q < total ? f0 + 256 * q : 0;  // clamped: unconditional loads
                const int row = f / nq4, k4 = (f % nq4) * 4;
                const int rc = row < n ? row : n - 1;
                v[q] = *reinterpret_cast<const float4 *>(xbase + s_xh[rc] + k4);
                u[q] = *reinterpret_cast<const float4 *>(xbase + s_xt[rc] + k4);
            }
#pragma unroll
            for (int q = 0; q < kBatch; ++q) {
                const int f = f0 + 256 * q;
                if (f < total) {
                    const int row = f / nq4, k4 = (f % nq4) * 4;
                    float4 x = sub_t ? make_float4(v[q].x - u[q].x, v[q].y - u[q].y, v[q].z - u[q].z, v[q].w - u[q].w) : v[q];
                    x = row < n ? scaled4(s_c[row], x) : make_float4(0.f, 0.f, 0.f, 0.f);
                    *reinterpret_cast<float4 *>(&sX[row * pitch + k4]) = x;
                }
            }
        }
    }
    const float *qbase = derived ? bwd_qbase(a.src) : a.qs;
    for (int c0 = 0; c0 < d; c0 += 256) {
        const int span = d - c0 < 256 ? d - c0 : 256;
        const int cw = ((span / 4 + 3) / 4) * 4;
        const int n0 = c0 + wave * cw;
        const int wcols = n0 >= c0 + span ? 0 : (c0 + span - n0 < cw ? c0 + span - n0 : cw);
        const bool colok = 4 * li < wcols;
        // this lane's columns of the q rows: one 128-bit load per position of its lane group, kept for all row blocks
        float4 bq[2][4];
        const float *qb = qbase + n0 + (colok ? 4 * li : 0);
#pragma unroll
        for (int q = 0; q < 2; ++q)
#pragma unroll
            for (int sidx = 0; sidx < 4; ++sidx) {
                const int i = 16 * q + 4 * kk + sidx;
                bq[q][sidx] = *reinterpret_cast<const float4 *>(qb + sOff[i < n ? i : n - 1]);
            }
        if constexpr (SIGN) {
#pragma unroll
            for (int q = 0; q < 2; ++q)
#pragma unroll
                for (int sidx = 0; sidx < 4; ++sidx) bq[q][sidx] = sgn4(bq[q][sidx]);
        }
        if (c0 == 0) __syncthreads();  // the staged rows (the loads above are in flight across the barrier)
        if (wcols <= 0) continue;
        for (int i0 = 0; i0 < d; i0 += 32) {
            floatx4 acc_lo[4], acc_hi[4];
#pragma unroll
            for (int e = 0; e < 4; ++e) acc_lo[e] = floatx4{0.f, 0.f, 0.f, 0.f}, acc_hi[e] = floatx4{0.f, 0.f, 0.f, 0.f};
            const bool ilo = i0 + li < d, ihi = i0 + 16 + li < d;
#pragma unroll
            for (int q = 0; q < 2; ++q) {
                if (q >= nq) break;
#pragma unroll
                for (int sidx = 0; sidx < 4; ++sidx) {
                    const int i = 16 * q + 4 * kk + sidx;
                    const float al = ilo ? sX[i * pitch + i0 + li] : 0.0f;
                    const float ah = ihi ? sX[i * pitch + i0 + 16 + li] : 0.0f;
                    const float b4[4] = {bq[q][sidx].x, bq[q][sidx].y, bq[q][sidx].z, bq[q][sidx].w};
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        acc_lo[e] = __builtin_amdgcn_mfma_f32_16x16x4f32(al, b4[e], acc_lo[e], 0, 0, 0);
                        acc_hi[e] = __builtin_amdgcn_mfma_f32_16x16x4f32(ah, b4[e], acc_hi[e], 0, 0, 0);
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
}

// dM[g][i][j] = sum_{p in group g} x[p][i] * q[p][j].  A work item is (chunk of <= 256 triples
// of one group, 32 rows i); it stages its 32 columns of the chunk's x rows in LDS (coefficients
// folded in), the four waves split the columns j and K runs over the chunk's triples.  Groups longer
// than one chunk write per-chunk partial matrices that are added up beside the segmented reduction
// (keeps the longest K loop at 16 supersteps).
__device__ __forceinline__ void transr_dm_item(const DmArgs &a, float *lds, int tile, int blk)
{
    const int d = a.d;
    const int i0 = blk * 32;
    const int g = a.plan.tile_seg[tile];
    const int s0 = a.plan.tile_p0[tile];
    const int seg_end = a.seg_offsets[g + 1];
    if (blk < 0) {  // a small group, whole, by this workgroup
        float *whole = a.dm + (int64_t)g * d * d;
        if (a.xs == nullptr && !a.src.rescal && a.src.norm_p == 1) transr_dm_small_body<true>(a, lds, s0, seg_end - s0, whole);
        else transr_dm_small_body<false>(a, lds, s0, seg_end - s0, whole);
        return;
    }
    const int s1 = s0 + kDmChunk < seg_end ? s0 + kDmChunk : seg_end;
    const int slot = a.plan.tile_part[tile];
    float *dst = slot >= 0 ? a.part + (int64_t)slot * d * d : a.dm + (int64_t)g * d * d;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int li = lane & 15, kk = lane >> 4;
    const bool two_blocks = i0 + 16 < d;
    const int n = s1 - s0, nq = (n + 15) / 16;
    const bool derived = a.xs == nullptr;

    // stage: thread i owns position s0 + i: the row's offset for the right operand, and the 32 columns
    // i0 .. i0 + 31 of its left operand (eight 128-bit loads, sixteen for TransR's two entity rows, all in
    // flight together), times the row's coefficient
    float *sX = lds;                                                      // [kDmChunk][kDmXP]
    int64_t *sOff = reinterpret_cast<int64_t *>(lds + kDmChunk * kDmXP);  // [kDmChunk]
    if (tid < 16 * nq) {
        const int p = s0 + (tid < n ? tid : n - 1);
        const float *ph, *pt;
        float coef = 1.0f;
        bool sub_t = false;
        if (derived) {
            const RowMeta m = bwd_row_meta(a.src, p, d);
            ph = a.src.ent + m.xh * d, pt = a.src.ent + m.xt * d;
            sOff[tid] = m.qoff, coef = m.coef, sub_t = !a.src.rescal;
        } else {
            ph = a.xs + (int64_t)p * d, pt = ph;
            sOff[tid] = (int64_t)p * d;
        }
        float4 v[8], u[8];
#pragma unroll
        for (int c = 0; c < 8; ++c) {
            const int col = i0 + 4 * c < d ? i0 + 4 * c : 0;  // clamped: unconditional loads, masked below
            v[c] = *reinterpret_cast<const float4 *>(ph + col);
        }
        if (sub_t) {  // uniform
#pragma unroll
            for (int c = 0; c < 8; ++c) u[c] = *reinterpret_cast<const float4 *>(pt + (i0 + 4 * c < d ? i0 + 4 * c : 0));
        } else {
#pragma unroll
            for (int c = 0; c < 8; ++c) u[c] = make_float4(0.f, 0.f, 0.f, 0.f);
        }
#pragma unroll
        for (int c = 0; c < 8; ++c) {
            float4 x = make_float4(v[c].x - u[c].x, v[c].y - u[c].y, v[c].z - u[c].z, v[c].w - u[c].w);
            x = (tid < n && i0 + 4 * c < d) ? scaled4(coef, x) : make_float4(0.f, 0.f, 0.f, 0.f);
            *reinterpret_cast<float4 *>(&sX[tid * kDmXP + 4 * c]) = x;
        }
    }
    __syncthreads();
    const float *qbase = derived ? bwd_qbase(a.src) : a.qs;
    const bool sign_rows = derived && !a.src.rescal && a.src.norm_p == 1;

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

        if (sign_rows) {
            if (two_blocks) dm_sweep<true, true>(qbase, sX, sOff, n, nq, n0, wcols, li, kk, acc_lo, acc_hi);
            else dm_sweep<false, true>(qbase, sX, sOff, n, nq, n0, wcols, li, kk, acc_lo, acc_hi);
        } else {
            if (two_blocks) dm_sweep<true, false>(qbase, sX, sOff, n, nq, n0, wcols, li, kk, acc_lo, acc_hi);
            else dm_sweep<false, false>(qbase, sX, sOff, n, nq, n0, wcols, li, kk, acc_lo, acc_hi);
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

static size_t dm_lds_bytes(int d)  // the staged left operand and its row offsets, or the thin groups' transposed rows
{
    const size_t item = sizeof(float) * kDmChunk * kDmXP + sizeof(int64_t) * kDmChunk, thin = sizeof(float) * 4 * (size_t)d;
    const size_t small = dm_small_fits(d) ? sizeof(float) * kDmSmallLdsFloats + sizeof(int64_t) * kDmSmall : 0;
    return item > thin ? (item > small ? item : small) : (thin > small ? thin : small);
}

// Item `it` of a dM pass: the (chunk, row block) items of the larger groups first (the long chains), then the
// small groups, then the thin ones.  False: past the end of the lists.
__device__ __forceinline__ bool transr_dm_work(const DmArgs &a, float *lds, int it, int n_long, int n_small, int n_thin)
{
    if (it < n_long) transr_dm_item(a, lds, a.plan.item_tile[it], a.plan.item_blk[it]);
    else if (it < n_long + n_small) transr_dm_item(a, lds, a.plan.item_tile[a.plan.max_items - 1 - (it - n_long)], -1);
    else if (it < n_long + n_small + n_thin) transr_thin_dm_body(a, lds, a.plan.thin_g[it - n_long - n_small]);
    else return false;
    return true;
}

// Grid: inspector workgroups (if any), kDmWgs workgroups of dM work, then the level-1 workgroups of the step's
// segmented reductions (entity rows from the dX launch's occurrence rows, relation rows from the forward's
// residual rows): they depend on nothing this kernel writes and run in the shadow of its long items.
__global__ __launch_bounds__(256, KGE_TR_OCC) void transr_dm_kernel(DmArgs a, FusedInsp fi, SegL1Rider sr)
{
    extern __shared__ __align__(16) float lds[];  // dm_lds_bytes(); inspector workgroups: their own need
    if (fused_insp_block(fi, reinterpret_cast<uint32_t *>(lds))) return;
    const int bid = (int)blockIdx.x - fi.blocks;
    if (bid >= kDmWgs) {
        seg_l1_rider_block(sr, bid - kDmWgs);
        return;
    }
    const int n_long = a.plan.num_items[0], n_small = a.plan.num_items[1], n_thin = a.plan.num_thin[0];
    for (int it = bid; transr_dm_work(a, lds, it, n_long, n_small, n_thin); it += kDmWgs)
        __syncthreads();  // the next item reuses the staging buffers
}

// An inspector step that rides with nothing: the fused entity inspection of a TransR / RESCAL step has
// four dependent steps and the step three kernels of its own (forward, dX, dM).
__global__ __launch_bounds__(256) void transr_insp_step_kernel(FusedInsp fi)
{
    extern __shared__ __align__(16) float lds[];
    (void)fused_insp_block(fi, reinterpret_cast<uint32_t *>(lds));
}

// dM of a split group = sum of its partial matrices (slot order = ascending chunk order); the sums
// ride in the segmented reduction's first launch
static SumRider dm_finish_rider(const DmArgs &a, int64_t max_split)
{
    SumRider r;
    r.part = a.part, r.out = a.dm;
    r.num = a.plan.num_split, r.seg = a.plan.split_seg, r.first = a.plan.split_first, r.cnt = a.plan.split_cnt;
    r.row_floats = (int64_t)a.d * a.d;
    r.max_sums = (int)max_split;
    return r;
}

// ---- host side -----------------------------------------------------------------------------
static size_t up256(size_t x) { return (x + 255) & ~size_t(255); }

struct RPlan {
    size_t off_plan, off_dplan, off_occ, off_part_e, off_part_r, off_dpart, total;
    int64_t tiles, dtiles, dsplit, dslots;
};

// (items > 0: a chunked plan with its work lists)
static size_t plan_ints(int64_t tiles, int64_t split, int64_t items = 0)
{
    return (size_t)(64 + 5 * tiles + 3 * split + (items > 0 ? tiles + 2 * items : 0) + 8);
}
static int dm_nib(int64_t d) { return (int)ceil_div(d, 32); }
static int dm_small_max(int64_t d) { return dm_small_fits((int)d) ? kDmSmall : kThin; }
static int64_t dm_item_cap(int64_t dtiles, int64_t d) { return dtiles * ceil_div(d, 32); }
static size_t dplan_ints(int64_t dtiles, int64_t dsplit, int64_t d) { return plan_ints(dtiles, dsplit, dm_item_cap(dtiles, d)); }

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
    p.off_dplan = o, o += up256(sizeof(int32_t) * dplan_ints(p.dtiles, p.dsplit, d));
    p.off_occ = o, o += up256(sizeof(float) * (size_t)(2 * B * d));
    p.off_part_e = o, o += up256(sizeof(float) * (size_t)seg_partial_floats(2 * B, d));
    p.off_part_r = o, o += up256(sizeof(float) * (size_t)seg_partial_floats(B, d));
    p.off_dpart = o, o += up256(sizeof(float) * (size_t)(p.dslots * d * d));
    p.total = o;
    return p;
}

static TilePlan plan_at(void *base, int64_t tiles, int64_t split, int64_t items = 0)
{
    int32_t *q = static_cast<int32_t *>(base);
    TilePlan p{};
    p.num_tiles = q, p.tile_seg = q + 64, p.tile_p0 = q + 64 + tiles;
    if (split > 0) {
        p.tile_part = q + 64 + 2 * tiles;
        p.num_split = q + 32;
        p.split_seg = q + 64 + 5 * tiles;
        p.split_first = p.split_seg + split;
        p.split_cnt = p.split_first + split;
        p.num_thin = q + 1, p.num_items = q + 2;
        p.thin_g = q + 64 + 5 * tiles + 3 * split;
        p.item_tile = p.thin_g + tiles;
        p.item_blk = p.item_tile + items;
        p.max_items = (int)items;
    } else {
        p.tile_end = q + 64 + 3 * tiles;
        p.tile_rid = q + 64 + 4 * tiles;
    }
    return p;
}
static TilePlan dplan_at(void *base, int64_t dtiles, int64_t dsplit, int64_t d)
{
    return plan_at(base, dtiles, dsplit, dm_item_cap(dtiles, d));
}

// The forward workspace holds both tile plans of the batch: the 32-triple tiles of the GEMM kernels
// and the chunked plan of the dM kernel.  A backward pass that is handed this workspace
// (kge_saved.fwd_workspace) finds its plans there and launches no plan kernel of its own.
static size_t fwd_plan_bytes(const kge_tables *tab, const kge_batch *bat)
{
    return up256(sizeof(int32_t) * plan_ints(max_tiles(tab, bat), 0));
}

static bool pad_path_ok(const kge_tables *, const kge_batch *);
static size_t transr_fwd_workspace_padded(const kge_tables *, const kge_batch *);
static size_t transr_bwd_workspace_padded(const kge_tables *, const kge_batch *);
static int launch_transr_fwd_padded(const kge_tables *, const kge_batch *, float *, float *, void *, size_t, hipStream_t);
static int launch_transr_plan_padded(const kge_tables *, const kge_batch *, void *, size_t, hipStream_t);
static int launch_transr_bwd_padded(const kge_tables *, const kge_batch *, const kge_saved *, const float *, const kge_grads *, void *,
                                    size_t, hipStream_t);

size_t transr_fwd_workspace(const kge_tables *tab, const kge_batch *bat)
{
    if (pad_path_ok(tab, bat)) return transr_fwd_workspace_padded(tab, bat);  // row width not a multiple of four
    const RPlan p = make_rplan(tab, bat);
    return fwd_plan_bytes(tab, bat) + up256(sizeof(int32_t) * dplan_ints(p.dtiles, p.dsplit, tab->dim));
}

// A launch with more than 64 KB of dynamic LDS has to be allowed per kernel first.
template <int MODE>
static int allow_lds(size_t bytes)
{
    if (bytes <= 64 * 1024) return KGE_OK;
    return hipFuncSetAttribute(reinterpret_cast<const void *>(&transr_gemm_kernel<MODE>),
                               hipFuncAttributeMaxDynamicSharedMemorySize, (int)kMaxGemmLds) == hipSuccess
               ? KGE_OK
               : KGE_ELAUNCH;
}

static size_t lds_with(const FusedInsp &fi, size_t own)
{
    return fi.blocks > 0 && (size_t)fi.lds_bytes > own ? (size_t)fi.lds_bytes : own;
}

// Whether the forward pass of this batch can also write the rows phi(y_b) Proj^T (kge_batch.back_rows).
bool back_rows_ok(const kge_tables *tab, const kge_batch *bat)
{
    return tab->model == KGE_TRANSR && bat->rel_insp && !bat->neg && !pad_path_ok(tab, bat) && mfma_path_ok(tab, bat) &&
           gemm_lds_bytes((int)tab->dim) <= kMaxGemmLds;
}

int launch_transr_fwd(const kge_tables *tab, const kge_batch *bat, float *pos, float *resid, void *workspace,
                      size_t workspace_bytes, hipStream_t st)
{
    if (bat->batch == 0) return KGE_OK;
    if (bat->back_rows && (!back_rows_ok(tab, bat) || !resid || !aligned16(bat->back_rows))) return KGE_EUNSUPPORTED;
    if (pad_path_ok(tab, bat) && workspace && workspace_bytes >= transr_fwd_workspace_padded(tab, bat))
        return launch_transr_fwd_padded(tab, bat, pos, resid, workspace, workspace_bytes, st);
    const bool rescal = tab->model == KGE_RESCAL;
    const bool grouped = mfma_path_ok(tab, bat) && workspace && workspace_bytes >= transr_fwd_workspace(tab, bat) &&
                         gemm_lds_bytes((int)tab->dim) <= kMaxGemmLds;
    if (bat->back_rows && !grouped) return KGE_EWORKSPACE;
    // fused entity inspection: its histogram step rides with the forward GEMM
    FusedInsp fi{};
    if (bat->fuse_inspection) {
        if (!grouped || !bat->insp_jobs || bat->neg) return KGE_EINVAL;
        const int rc = plan_fused_inspection(bat->insp_jobs, 1, 0, &fi);
        if (rc) return rc;
    }
    if (!grouped) {
        const int rc = launch_score_pos(tab, bat, pos, resid, nullptr, st);
        timeline_mark(bat->timeline, st, "score_pos_kernel");
        return rc;
    }
    const kge_inspection *ri = bat->rel_insp;
    const int64_t tiles = max_tiles(tab, bat);
    TilePlan plan = plan_at(workspace, tiles, 0);
    const RPlan rp = make_rplan(tab, bat);
    TilePlan dplan = dplan_at(static_cast<char *>(workspace) + fwd_plan_bytes(tab, bat), rp.dtiles, rp.dsplit, tab->dim);
    if (!bat->plans_ready)
        hipLaunchKernelGGL(transr_plan_kernel, dim3(2), dim3(1024), 0, st, ri->num_unique, ri->seg_offsets, ri->unique_ids, plan,
                           kTM, dplan, kDmChunk, dm_nib(tab->dim), dm_small_max(tab->dim));
    GemmArgs a{tab->ent, tab->rel, tab->aux, bat->h, bat->r, bat->t, ri->perm, ri->seg_offsets, ri->num_unique, ri->unique_ids,
               plan, nullptr, nullptr, pos, resid, nullptr, nullptr, (int)tab->dim, tab->norm_p, thin_groups(tab, bat), (int)tiles,
               BwdSrc{}, bat->back_rows};
    size_t own = gemm_lds_bytes((int)tab->dim);
    if (a.back && thin_both_lds_bytes((int)tab->dim) > own) own = thin_both_lds_bytes((int)tab->dim);
    const size_t lds = lds_with(fi, own);
    const dim3 grid((unsigned)(tiles + a.thin_groups + fi.blocks));
    if (a.back) {
        if (lds > 64 * 1024 && hipFuncSetAttribute(reinterpret_cast<const void *>(&transr_fwd_back_kernel),
                                                   hipFuncAttributeMaxDynamicSharedMemorySize, (int)kMaxGemmLds) != hipSuccess)
            return KGE_ELAUNCH;
        hipLaunchKernelGGL(transr_fwd_back_kernel, grid, dim3(256), lds, st, a, fi);
    } else {
        if (const int rc = rescal ? allow_lds<1>(lds) : allow_lds<0>(lds)) return rc;
        if (rescal)
            hipLaunchKernelGGL(transr_gemm_kernel<1>, grid, dim3(256), lds, st, a, fi);
        else
            hipLaunchKernelGGL(transr_gemm_kernel<0>, grid, dim3(256), lds, st, a, fi);
    }
    timeline_mark(bat->timeline, st, a.back ? "transr_plan_kernel + transr_fwd_back_kernel"
                                            : "transr_plan_kernel + transr_gemm_kernel<fwd>");
    KGE_CHECK_LAUNCH();
    return KGE_OK;
}

// RESCAL with corrupted heads: the pair score E[h'] . (Proj[r] E[t]) needs the rows u_b = E[t_b] Proj[r_b]^T.  Same
// grouped pass as dX with E[t] as its upstream rows and coefficient 1; the plans are the ones the forward call of
// the positives left in `workspace`.
int launch_rescal_head_rows(const kge_tables *tab, const kge_batch *bat, float *u, void *workspace, size_t workspace_bytes,
                            hipStream_t st)
{
    if (bat->batch == 0) return KGE_OK;
    if (tab->model != KGE_RESCAL || !bat->rel_insp || !u || !aligned16(u)) return KGE_EINVAL;
    if (pad_path_ok(tab, bat) || !mfma_path_ok(tab, bat) || gemm_lds_bytes((int)tab->dim) > kMaxGemmLds) return KGE_EUNSUPPORTED;
    if (!workspace || workspace_bytes < transr_fwd_workspace(tab, bat)) return KGE_EWORKSPACE;
    const kge_inspection *ri = bat->rel_insp;
    const int d = (int)tab->dim;
    const int64_t tiles = max_tiles(tab, bat);
    TilePlan plan = plan_at(workspace, tiles, 0);
    const BwdSrc src{tab->ent, nullptr, nullptr, nullptr, bat->h, bat->t, ri->perm, tab->norm_p, 1, nullptr, 1};
    GemmArgs ga{tab->ent, tab->rel, tab->aux, bat->h, bat->r, bat->t, ri->perm, ri->seg_offsets, ri->num_unique, ri->unique_ids,
                plan, nullptr, nullptr, nullptr, nullptr, u, nullptr, d, tab->norm_p, thin_groups(tab, bat), (int)tiles, src};
    if (const int rc = allow_lds<2>(gemm_lds_bytes(d))) return rc;
    hipLaunchKernelGGL(transr_gemm_kernel<2>, dim3((unsigned)(tiles + ga.thin_groups)), dim3(256), gemm_lds_bytes(d), st, ga, FusedInsp{});
    timeline_mark(bat->timeline, st, "transr_gemm_kernel<head rows>");
    KGE_CHECK_LAUNCH();
    return KGE_OK;
}

// The tile plans alone (what launch_transr_fwd builds first), for callers that plan a batch ahead.
int launch_transr_plan(const kge_tables *tab, const kge_batch *bat, void *workspace, size_t workspace_bytes, hipStream_t st)
{
    if (bat->batch == 0) return KGE_OK;
    if (bat->neg && tab->model == KGE_TRANSR) return KGE_EUNSUPPORTED;  // TransR's shared-negative path plans its own row list
    if (pad_path_ok(tab, bat)) return launch_transr_plan_padded(tab, bat, workspace, workspace_bytes, st);
    if (!mfma_path_ok(tab, bat) || gemm_lds_bytes((int)tab->dim) > kMaxGemmLds) return KGE_EUNSUPPORTED;
    if (!workspace || workspace_bytes < transr_fwd_workspace(tab, bat)) return KGE_EWORKSPACE;
    const kge_inspection *ri = bat->rel_insp;
    const RPlan rp = make_rplan(tab, bat);
    TilePlan plan = plan_at(workspace, max_tiles(tab, bat), 0);
    TilePlan dplan = dplan_at(static_cast<char *>(workspace) + fwd_plan_bytes(tab, bat), rp.dtiles, rp.dsplit, tab->dim);
    hipLaunchKernelGGL(transr_plan_kernel, dim3(2), dim3(1024), 0, st, ri->num_unique, ri->seg_offsets, ri->unique_ids, plan, kTM,
                       dplan, kDmChunk, dm_nib(tab->dim), dm_small_max(tab->dim));
    KGE_CHECK_LAUNCH();
    return KGE_OK;
}

// ---- RESCAL with shared negatives that replace the tail ---------------------------------------------
// score(b, k) = (E[h_b] Proj[r_b]) . E[n_k] = q_b . E[n_k]: the negatives need no projection at all.  Forward:
// the grouped pass leaves q_b (and the positive score q_b . E[t_b]); the pair scores are the dot-product
// tile of DistMult with q_b as the query rows.  Backward: the gradient tiles give the negatives' rows and
// G_b = sum_k dneg[b][k] E[n_k] = dL/dq_b from the pairs; with the positive's own term the upstream row of
// the projected vector is Q_b = dpos[b] E[t_b] + G_b, and dX = Q M^T, dM = X^T Q (X = E[h]) run as the
// grouped passes over B rows instead of B (1 + N) flattened triples.
int launch_rescal_neg_tiles(const kge_tables *, const kge_batch *, const float *, const float *, float *, float *, hipStream_t);

struct RescalNegPlan {
    size_t off_plan, off_dplan, off_xs, off_qs, off_g0, off_occ, off_part_e, off_dpart, total;
    int64_t tiles, dtiles, dsplit, dslots, nn;
};

static RescalNegPlan make_rescal_neg_plan(const kge_tables *tab, const kge_batch *bat)
{
    RescalNegPlan p{};
    const RPlan r = make_rplan(tab, bat);
    const int64_t B = bat->batch, d = tab->dim;
    p.tiles = r.tiles, p.dtiles = r.dtiles, p.dsplit = r.dsplit, p.dslots = r.dslots;
    p.nn = bat->chunk > 0 ? (B / bat->chunk) * bat->n_neg : 0;
    size_t o = 0;
    auto take = [&](size_t bytes) {
        const size_t at = o;
        o += up256(bytes > 0 ? bytes : 1);
        return at;
    };
    p.off_plan = take(sizeof(int32_t) * plan_ints(p.tiles, 0));
    p.off_dplan = take(sizeof(int32_t) * dplan_ints(p.dtiles, p.dsplit, d));
    p.off_xs = take(sizeof(float) * (size_t)(B * d));
    p.off_qs = take(sizeof(float) * (size_t)(B * d));
    p.off_g0 = take(sizeof(float) * (size_t)(B * d));
    p.off_occ = take(sizeof(float) * (size_t)((2 * B + p.nn) * d));
    p.off_part_e = take(sizeof(float) * (size_t)seg_partial_floats(2 * B + p.nn, d));
    p.off_dpart = take(sizeof(float) * (size_t)(p.dslots * d * d));
    p.total = o;
    return p;
}

size_t transr_bwd_workspace(const kge_tables *tab, const kge_batch *bat)
{
    if (tab->model == KGE_RESCAL && bat->neg) return make_rescal_neg_plan(tab, bat).total;
    if (pad_path_ok(tab, bat)) return transr_bwd_workspace_padded(tab, bat);
    return make_rplan(tab, bat).total;
}

// One wave per sorted position p (triple b = perm[p]).  Replaced tails: xs[p] = E[h], qs[p] = g E[t] + G[b],
// occ_o[b] = g v[b] (the tail's occurrence row, v = E[h] Proj[r]).  Replaced heads (head != 0): xs[p] = g E[h] + G[b],
// qs[p] = E[t], occ_o[b] = g u[b] (the head's occurrence row, u = Proj[r] E[t]).
__global__ __launch_bounds__(256) void rescal_neg_prep_kernel(const float *ent, const int64_t *h, const int64_t *t, const int32_t *perm,
                                                              const float *dpos, const float *G, const float *resid, float *xs,
                                                              float *qs, float *occ_o, int64_t B, int d, int head)
{
    const int lane = threadIdx.x & 63;
    const int64_t p = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (p >= B) return;
    const int b = perm[p];
    const float g = dpos ? dpos[b] : 0.0f;
    const float *eh = ent + h[b] * (int64_t)d, *et = ent + t[b] * (int64_t)d;
    for (int j = lane * 4; j < d; j += 256) {
        const float4 vh = *reinterpret_cast<const float4 *>(eh + j), vt = *reinterpret_cast<const float4 *>(et + j);
        const float4 ve = *reinterpret_cast<const float4 *>(resid + (int64_t)b * d + j);
        const float4 vg = G ? *reinterpret_cast<const float4 *>(G + (int64_t)b * d + j) : make_float4(0.f, 0.f, 0.f, 0.f);
        if (head) {  // uniform
            *reinterpret_cast<float4 *>(xs + p * d + j) = make_float4(fmaf(g, vh.x, vg.x), fmaf(g, vh.y, vg.y), fmaf(g, vh.z, vg.z), fmaf(g, vh.w, vg.w));
            *reinterpret_cast<float4 *>(qs + p * d + j) = vt;
        } else {
            *reinterpret_cast<float4 *>(xs + p * d + j) = vh;
            *reinterpret_cast<float4 *>(qs + p * d + j) = make_float4(fmaf(g, vt.x, vg.x), fmaf(g, vt.y, vg.y), fmaf(g, vt.z, vg.z), fmaf(g, vt.w, vg.w));
        }
        *reinterpret_cast<float4 *>(occ_o + (int64_t)b * d + j) = scaled4(g, ve);
    }
}

__global__ void rescal_fill_zero_kernel(float *p, int64_t n)
{
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x) p[i] = 0.0f;
}

int launch_rescal_neg_bwd(const kge_tables *tab, const kge_batch *bat, const kge_saved *saved, const float *dpos,
                                 const float *dneg, const kge_grads *grads, void *workspace, size_t workspace_bytes, hipStream_t st)
{
    const bool head = bat->neg_mode == KGE_NEG_HEAD;
    if (!mfma_path_ok(tab, bat) || gemm_lds_bytes((int)tab->dim) > kMaxGemmLds) return KGE_EUNSUPPORTED;
    if (bat->fuse_inspection) return KGE_EINVAL;
    if (!saved->residual || !aligned16(saved->residual) || !grads->aux_rows || !grads->ent_rows) return KGE_EINVAL;
    if (grads->aux_factor_max != 0) return KGE_EUNSUPPORTED;
    const RescalNegPlan p = make_rescal_neg_plan(tab, bat);
    if (!workspace || workspace_bytes < p.total || !aligned16(workspace)) return KGE_EWORKSPACE;
    if (bat->ent_insp->n != 2 * bat->batch + p.nn) return KGE_ESHAPE;
    const int64_t B = bat->batch;
    const int d = (int)tab->dim;
    char *ws = static_cast<char *>(workspace);
    float *xs = reinterpret_cast<float *>(ws + p.off_xs), *qs = reinterpret_cast<float *>(ws + p.off_qs);
    float *g0 = reinterpret_cast<float *>(ws + p.off_g0), *occ = reinterpret_cast<float *>(ws + p.off_occ);
    const kge_inspection *ri = bat->rel_insp;
    if (dneg) {
        const int rc = launch_rescal_neg_tiles(tab, bat, saved->residual, dneg, g0, occ + 2 * B * d, st);
        timeline_mark(bat->timeline, st, "bwd_tile_kernel");
        if (rc) return rc;
    } else if (p.nn > 0) {  // no upstream gradient on the pairs: the negatives' occurrence rows are zero
        hipLaunchKernelGGL(rescal_fill_zero_kernel, dim3(1024), dim3(256), 0, st, occ + 2 * B * d, p.nn * d);
    }
    // (occurrence rows: [h of the B positives | t of the B positives | negatives])
    hipLaunchKernelGGL(rescal_neg_prep_kernel, dim3((unsigned)ceil_div(B, 4)), dim3(256), 0, st, tab->ent, bat->h, bat->t, ri->perm, dpos,
                       dneg ? g0 : nullptr, saved->residual, xs, qs, head ? occ : occ + B * d, B, d, head ? 1 : 0);
    TilePlan plan = plan_at(ws + p.off_plan, p.tiles, 0), dplan = dplan_at(ws + p.off_dplan, p.dtiles, p.dsplit, d);
    hipLaunchKernelGGL(transr_plan_kernel, dim3(2), dim3(1024), 0, st, ri->num_unique, ri->seg_offsets, ri->unique_ids, plan, kTM, dplan,
                       kDmChunk, dm_nib(d), dm_small_max(d));
    if (head) {
        // the tails' rows: (g E[h] + G) Proj[r], the forward product on rows given as an array, written per triple
        GemmArgs ga{tab->ent, tab->rel, tab->aux, bat->h, bat->r, bat->t, ri->perm, ri->seg_offsets, ri->num_unique, ri->unique_ids,
                    plan, xs, nullptr, nullptr, occ + B * d, nullptr, nullptr, d, tab->norm_p, thin_groups(tab, bat), (int)p.tiles,
                    BwdSrc{}};
        if (const int rc = allow_lds<1>(gemm_lds_bytes(d))) return rc;
        hipLaunchKernelGGL(transr_gemm_kernel<1>, dim3((unsigned)(p.tiles + ga.thin_groups)), dim3(256), gemm_lds_bytes(d), st, ga,
                           FusedInsp{});
    } else {
        GemmArgs ga{tab->ent, tab->rel, tab->aux, bat->h, bat->r, bat->t, ri->perm, ri->seg_offsets, ri->num_unique, ri->unique_ids,
                    plan, qs, nullptr, nullptr, nullptr, occ, nullptr, d, tab->norm_p, thin_groups(tab, bat), (int)p.tiles, BwdSrc{}};
        if (const int rc = allow_lds<2>(gemm_lds_bytes(d))) return rc;
        hipLaunchKernelGGL(transr_gemm_kernel<2>, dim3((unsigned)(p.tiles + ga.thin_groups)), dim3(256), gemm_lds_bytes(d), st, ga,
                           FusedInsp{});
    }
    timeline_mark(bat->timeline, st, "transr_gemm_kernel<dX>");
    // dProj[r][i][j] = sum over the group of xs[i] qs[j] in both modes
    DmArgs da{xs, qs, ri->seg_offsets, dplan, grads->aux_rows, reinterpret_cast<float *>(ws + p.off_dpart), d, ri->num_unique,
              BwdSrc{}, nullptr, nullptr, 0};
    hipLaunchKernelGGL(transr_dm_kernel, dim3((unsigned)kDmWgs), dim3(256), dm_lds_bytes(d), st, da, FusedInsp{}, SegL1Rider{});
    timeline_mark(bat->timeline, st, "transr_dm_kernel");
    KGE_CHECK_LAUNCH();
    if (bat->insp_ready && hipStreamWaitEvent(st, reinterpret_cast<hipEvent_t>(bat->insp_ready), 0) != hipSuccess)
        return KGE_ELAUNCH;
    const SegJob jobs[1] = {{occ, bat->ent_insp, d, grads->ent_rows, reinterpret_cast<float *>(ws + p.off_part_e), false}};
    const SumRider finish = dm_finish_rider(da, p.dsplit);
    return launch_seg_reduce_jobs(jobs, 1, st, bat->timeline, &finish);
}

int launch_transr_bwd(const kge_tables *tab, const kge_batch *bat, const kge_saved *saved, const float *dpos,
                      const kge_grads *grads, void *workspace, size_t workspace_bytes, hipStream_t st)
{
    const bool rescal = tab->model == KGE_RESCAL;
    if (bat->neg) return KGE_EUNSUPPORTED;  // (shared negatives: launch_transr_neg_bwd / launch_rescal_neg_bwd)
    if (saved->back_rows && !back_rows_ok(tab, bat)) return KGE_EINVAL;  // (no forward pass writes them for this batch)
    if (pad_path_ok(tab, bat)) return launch_transr_bwd_padded(tab, bat, saved, dpos, grads, workspace, workspace_bytes, st);
    if (!mfma_path_ok(tab, bat) || gemm_lds_bytes((int)tab->dim) > kMaxGemmLds) return KGE_EUNSUPPORTED;
    if (!saved->residual || !grads->aux_rows || !grads->ent_rows) return KGE_EINVAL;
    if (!rescal && (!grads->rel_rows || (tab->norm_p == 2 && !saved->pos))) return KGE_EINVAL;
    // factored projection gradients of the small groups: both arrays, 16-byte aligned, at most kThin rows
    const bool factored = grads->aux_factor_max > 0;
    if (grads->aux_factor_max < 0 || grads->aux_factor_max > kThin) return KGE_EINVAL;
    if (factored && (!grads->aux_x || !grads->aux_q || !aligned16(grads->aux_x) || !aligned16(grads->aux_q))) return KGE_EINVAL;
    if (!aligned16(saved->residual)) return KGE_EINVAL;
    const RPlan p = make_rplan(tab, bat);
    if (!workspace || workspace_bytes < p.total) return KGE_EWORKSPACE;
    if (bat->ent_insp->n != 2 * bat->batch) return KGE_ESHAPE;
    const int64_t B = bat->batch;
    const int d = (int)tab->dim;
    char *ws = static_cast<char *>(workspace);
    float *occ = reinterpret_cast<float *>(ws + p.off_occ);
    const kge_inspection *ri = bat->rel_insp;
    // the plans: left behind by the forward pass, or built here
    const bool have_plans = saved->fwd_workspace && saved->fwd_workspace_bytes >= transr_fwd_workspace(tab, bat);
    char *pbase = have_plans ? static_cast<char *>(const_cast<void *>(saved->fwd_workspace)) : nullptr;
    TilePlan plan = have_plans ? plan_at(pbase, p.tiles, 0) : plan_at(ws + p.off_plan, p.tiles, 0);
    TilePlan dplan = have_plans ? dplan_at(pbase + fwd_plan_bytes(tab, bat), p.dtiles, p.dsplit, d)
                                : dplan_at(ws + p.off_dplan, p.dtiles, p.dsplit, d);

    // fused entity inspection (its histogram rode with the forward GEMM): first digit pass in a launch
    // of its own, second with the dX GEMM, dedup with dM
    FusedInsp f1{}, f2{}, f3{};
    if (bat->fuse_inspection) {
        if (!bat->insp_jobs) return KGE_EINVAL;
        int rc;
        if ((rc = plan_fused_inspection(bat->insp_jobs, 1, 1, &f1))) return rc;
        if ((rc = plan_fused_inspection(bat->insp_jobs, 1, 2, &f2))) return rc;
        if ((rc = plan_fused_inspection(bat->insp_jobs, 1, 3, &f3))) return rc;
        hipLaunchKernelGGL(transr_insp_step_kernel, dim3((unsigned)f1.blocks), dim3(256), lds_with(f1, 0), st, f1);
        timeline_mark(bat->timeline, st, "inspector step");
    }
    if (!have_plans)
        hipLaunchKernelGGL(transr_plan_kernel, dim3(2), dim3(1024), 0, st, ri->num_unique, ri->seg_offsets, ri->unique_ids, plan, kTM,
                           dplan, kDmChunk, dm_nib(d), dm_small_max(d));
    // Upstream rows q and left operands x are formed inside the two kernels from the forward pass's rows
    // (BwdSrc); RESCAL's tail occurrence rows g * v come out of the dX kernel's staging.
    const BwdSrc src{tab->ent, saved->residual, dpos, saved->pos, bat->h, bat->t, ri->perm, tab->norm_p, rescal ? 1 : 0,
                     rescal ? occ + B * d : nullptr};
    // dX = Q M^T -> occurrence rows of h (and -dX for t)
    GemmArgs ga{tab->ent, tab->rel, tab->aux, bat->h, bat->r, bat->t, ri->perm, ri->seg_offsets, ri->num_unique, ri->unique_ids,
                plan, nullptr, nullptr, nullptr, nullptr, occ, rescal ? nullptr : occ + B * d, d, tab->norm_p, thin_groups(tab, bat),
                (int)p.tiles, src};
    // dM = X^T Q per relation group
    DmArgs da{nullptr, nullptr, ri->seg_offsets, dplan, grads->aux_rows, reinterpret_cast<float *>(ws + p.off_dpart), d,
              ri->num_unique, src, factored ? grads->aux_x : nullptr, factored ? grads->aux_q : nullptr, grads->aux_factor_max};
    // With the forward pass's rows z_b = phi(y_b) Proj^T at hand (kge_saved.back_rows) the entity gradients are
    // +-coef_b z_b and no kernel reads the projections again: the reduction scales the rows as it loads them.
    const bool have_back = saved->back_rows != nullptr;
    if (have_back && (rescal || !aligned16(saved->back_rows))) return KGE_EINVAL;
    if (!have_back) {
        if (const int rc = allow_lds<2>(lds_with(f2, gemm_lds_bytes(d)))) return rc;
        hipLaunchKernelGGL(transr_gemm_kernel<2>, dim3((unsigned)(p.tiles + ga.thin_groups + f2.blocks)), dim3(256),
                           lds_with(f2, gemm_lds_bytes(d)), st, ga, f2);
        timeline_mark(bat->timeline, st, "transr_gemm_kernel<dX>");
    } else if (f2.blocks > 0) {  // the inspector step that would have ridden with dX
        hipLaunchKernelGGL(transr_insp_step_kernel, dim3((unsigned)f2.blocks), dim3(256), lds_with(f2, 0), st, f2);
        timeline_mark(bat->timeline, st, "inspector step");
    }
    // entity rows from the h / t occurrence rows; dR[g] = sum of the group's upstream rows, formed from the
    // residual rows as the reduction loads them (scale dpos or dpos / pos, sign for L1).  Level 1 of both rides
    // in the dM launch, level 2 (with the sums that finish the split groups' dM) follows it.
    SegJob jobs[2] = {{occ, bat->ent_insp, d, grads->ent_rows, reinterpret_cast<float *>(ws + p.off_part_e), false},
                      {saved->residual, ri, d, grads->rel_rows, reinterpret_cast<float *>(ws + p.off_part_r), false}};
    jobs[1].scaled = true, jobs[1].sign_rows = tab->norm_p == 1;
    jobs[1].scale_num = dpos, jobs[1].scale_den = tab->norm_p == 2 ? saved->pos : nullptr;
    if (have_back) {  // occurrence i < B is +coef z_i (the head's), occurrence B + i is -coef z_i (the tail's)
        jobs[0].occ = saved->back_rows, jobs[0].scaled = true, jobs[0].wrap = B;
        jobs[0].scale_num = dpos, jobs[0].scale_den = tab->norm_p == 2 ? saved->pos : nullptr;
    }
    const int n_jobs = rescal ? 1 : 2;
    if (bat->insp_ready && hipStreamWaitEvent(st, reinterpret_cast<hipEvent_t>(bat->insp_ready), 0) != hipSuccess)
        return KGE_ELAUNCH;
    // (not when the last step of a fused entity inspection rides in this launch: level 1 reads its result)
    const bool ride = f3.blocks == 0;
    const SegL1Rider sr = ride ? plan_seg_l1_rider(jobs, n_jobs) : SegL1Rider{};
    hipLaunchKernelGGL(transr_dm_kernel, dim3((unsigned)(kDmWgs + f3.blocks + sr.blocks())), dim3(256), lds_with(f3, dm_lds_bytes(d)), st,
                       da, f3, sr);
    timeline_mark(bat->timeline, st, "transr_dm_kernel");
    KGE_CHECK_LAUNCH();
    const SumRider finish = dm_finish_rider(da, p.dsplit);
    return launch_seg_reduce_jobs(jobs, n_jobs, st, bat->timeline, &finish, ride);
}

#include "transr_neg.hpp"
#include "transr_pad.hpp"

}  // namespace kge
