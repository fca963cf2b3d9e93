// TransR with shared negatives: every negative is projected once per (relation, chunk) group.
//
// The reference defines the shared-negative TransR score on the flattened batch * blocksize
// triples (apps/examples/examples.py:1447-1480: the views of vh, vt, vr, mr are all expanded to
// output_size rows before bvm), i.e. one vector x matrix product per (positive, negative) pair.
// With x_b the entity the positive keeps (the head; the tail when the negatives replace heads),
// sigma = +1 / -1 and n_k the chunk's negatives, the pair residual splits into two projections,
//     (x_b - n_k) M_r + R_r   =   a_b - P_(g,k),      a_b = x_b M_r + sigma R_r,   P_(g,k) = n_k M_r
// (head mode: (n_k - x_b) M_r + R_r = -(a_b - P_(g,k)), same norm), and P only depends on the
// GROUP g = (relation, chunk) of the positive.  So the batch is turned into one list of rows to
// project, ordered by relation,
//     relation u :  [ positives' own rows (h - t) | their a rows | N rows per group of u ]
// which the grouped matrix-core kernels of transr.hip project in ONE pass (list mode), and small
// per-pair kernels form the scores ||a_b - P_(g(b),k)|| and, backward, the gradients with respect
// to the a and P rows; the chain through the projections (dX = Q M^T, dM = X^T Q) is again one
// grouped pass over the same list.  The matrix-core work drops from B (1 + N) rows to
// 2 B + G N rows, G = number of distinct (relation, chunk) pairs of the batch.
//
// This file is included by transr.hip (inside namespace kge) below the grouped kernels.

constexpr int kNegSeg = 8;  // sorted positions per wave of the P-row gradient sum

struct NegShape {
    int64_t B, N, C, n_chunks, NN, d, U_cap, G_cap, L_cap;
    int64_t tiles, dtiles, dsplit, dslots;
};

static NegShape neg_shape(const kge_tables *tab, const kge_batch *bat)
{
    NegShape s{};
    s.B = bat->batch, s.N = bat->n_neg, s.C = bat->chunk, s.d = tab->dim;
    s.n_chunks = s.C > 0 ? s.B / s.C : 0;
    s.NN = s.n_chunks * s.N;
    s.U_cap = s.B < tab->n_rel ? s.B : tab->n_rel;
    const int64_t pairs = tab->n_rel * s.n_chunks;
    s.G_cap = s.B < pairs ? s.B : pairs;
    s.L_cap = 2 * s.B + s.G_cap * s.N;
    s.tiles = s.U_cap + s.L_cap / kTM + 1;
    s.dtiles = s.U_cap + s.L_cap / kDmChunk + 1;
    s.dsplit = s.L_cap / kDmChunk + 1;
    s.dslots = 2 * (s.L_cap / kDmChunk) + 2;
    return s;
}

// forward workspace: the group inspection, the row list, both tile plans and the projected rows;
// kge_score_bwd finds them through kge_saved.fwd_workspace
struct NegFwdLayout {
    size_t keys, knum, kuniq, kseg, kperm, kinv, ksseg, kws, kws_bytes;
    size_t gstart, segl, rowpos, rowa, rowp, hl, tl, rsl, plan, dplan, y, total;
};

static NegFwdLayout neg_fwd_layout(const kge_tables *tab, const NegShape &s)
{
    NegFwdLayout l{};
    size_t o = 0;
    auto take = [&](size_t bytes) {
        const size_t at = o;
        o += up256(bytes > 0 ? bytes : 1);
        return at;
    };
    l.keys = take(sizeof(int64_t) * s.B);
    l.knum = take(sizeof(int32_t));
    l.kuniq = take(sizeof(int64_t) * s.B);
    l.kseg = take(sizeof(int32_t) * (s.B + 1));
    l.kperm = take(sizeof(int32_t) * s.B);
    l.kinv = take(sizeof(int32_t) * s.B);
    l.ksseg = take(sizeof(int32_t) * s.B);
    l.kws_bytes = kge_inspect_workspace(s.B, tab->n_rel * s.n_chunks);
    l.kws = take(l.kws_bytes);
    l.gstart = take(sizeof(int32_t) * (s.U_cap + 1));
    l.segl = take(sizeof(int32_t) * (s.U_cap + 1));
    l.rowpos = take(sizeof(int32_t) * s.B);
    l.rowa = take(sizeof(int32_t) * s.B);
    l.rowp = take(sizeof(int32_t) * s.G_cap);
    l.hl = take(sizeof(int64_t) * s.L_cap);
    l.tl = take(sizeof(int64_t) * s.L_cap);
    l.rsl = take(sizeof(float) * s.L_cap);
    l.plan = take(sizeof(int32_t) * plan_ints(s.tiles, 0));
    l.dplan = take(sizeof(int32_t) * dplan_ints(s.dtiles, s.dsplit, s.d));
    l.y = take(sizeof(float) * (size_t)(s.L_cap * s.d));
    l.total = o;
    return l;
}

struct NegBwdLayout {
    size_t xl, ql, dxl, occ, qr, glist, gcount, ppart, part_e, part_r, dpart, total;
};

static NegBwdLayout neg_bwd_layout(const NegShape &s)
{
    NegBwdLayout l{};
    size_t o = 0;
    auto take = [&](size_t bytes) {
        const size_t at = o;
        o += up256(bytes > 0 ? bytes : 1);
        return at;
    };
    const size_t rows = sizeof(float) * (size_t)(s.L_cap * s.d);
    l.xl = take(rows), l.ql = take(rows), l.dxl = take(rows);
    l.occ = take(sizeof(float) * (size_t)((2 * s.B + s.NN) * s.d));
    l.qr = take(sizeof(float) * (size_t)(s.B * s.d));
    l.glist = take(sizeof(int32_t) * s.B);
    l.gcount = take(sizeof(int32_t) * s.n_chunks);
    l.ppart = take(sizeof(float) * (size_t)(ceil_div(s.B, kNegSeg) * s.N * 2 * s.d));
    l.part_e = take(sizeof(float) * (size_t)seg_partial_floats(2 * s.B + s.NN, s.d));
    l.part_r = take(sizeof(float) * (size_t)seg_partial_floats(s.B, s.d));
    l.dpart = take(sizeof(float) * (size_t)(s.dslots * s.d * s.d));
    l.total = o;
    return l;
}

// Everything the small kernels index with (device pointers into the forward workspace).
struct NegIdx {
    const int64_t *h, *r, *t, *neg;
    // inspection of the relation ids (the caller's rel_insp)
    const int32_t *r_num, *r_seg, *r_perm, *r_inv, *r_sseg;
    const int64_t *r_uniq;
    // inspection of the group keys r * n_chunks + chunk
    int64_t *keys;
    const int32_t *k_num, *k_seg, *k_perm, *k_inv;
    const int64_t *k_uniq;
    int32_t *gstart, *segl, *rowpos, *rowa, *rowp;
    int64_t *hl, *tl;
    float *rsl;
    int64_t B, N, C, n_chunks, G_cap;
    int d, head;
};

__global__ void tneg_keys_kernel(NegIdx x)
{
    const int64_t b = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (b < x.B) x.keys[b] = x.r[b] * x.n_chunks + b / x.C;
}

// gstart[u]: index of relation u's first group in the (relation-major) key order; segl[u]: first
// list row of relation u = 2 positions per positive of the smaller relations + N per group
__global__ void tneg_gstart_kernel(NegIdx x)
{
    const int u = blockIdx.x * blockDim.x + threadIdx.x;
    const int U = x.r_num[0], G = x.k_num[0];
    if (u > U) return;
    if (u == U) {
        x.gstart[U] = G;
        x.segl[U] = (int32_t)(2 * x.B + x.N * G);
        return;
    }
    const int64_t target = x.r_uniq[u] * x.n_chunks;
    int lo = 0, hi = G;  // first group whose key is >= target
    while (lo < hi) {
        const int mid = (lo + hi) >> 1;
        if (x.k_uniq[mid] < target) lo = mid + 1;
        else hi = mid;
    }
    x.gstart[u] = lo;
    x.segl[u] = (int32_t)(2 * x.r_seg[u] + x.N * lo);
}

// The list rows (entity to project, entity to subtract or -1, factor of the relation row) and where
// each positive's and each group's rows sit.
__global__ void tneg_list_kernel(NegIdx x)
{
    const int64_t total = x.B + x.G_cap * x.N;
    const int G = x.k_num[0];
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (int64_t)gridDim.x * blockDim.x) {
        if (i < x.B) {
            const int p = (int)i;  // position in relation order
            const int u = x.r_sseg[p], s0 = x.r_seg[u], n_u = x.r_seg[u + 1] - s0, j = p - s0;
            const int b = x.r_perm[p];
            const int base = x.segl[u];
            const int64_t hb = x.h[b], tb = x.t[b];
            x.hl[base + j] = hb, x.tl[base + j] = tb, x.rsl[base + j] = 1.0f;
            x.rowpos[b] = base + j;
            const int ra = base + n_u + j;
            x.hl[ra] = x.head ? tb : hb, x.tl[ra] = -1, x.rsl[ra] = x.head ? -1.0f : 1.0f;
            x.rowa[b] = ra;
        } else {
            const int64_t q = i - x.B;
            const int g = (int)(q / x.N), k = (int)(q % x.N);
            if (g >= G) continue;
            const int brep = x.k_perm[x.k_seg[g]];  // any positive of the group names its relation and chunk
            const int u = x.r_inv[brep];
            const int64_t c = brep / x.C;
            const int n_u = x.r_seg[u + 1] - x.r_seg[u];
            const int base = x.segl[u] + 2 * n_u + (g - x.gstart[u]) * (int)x.N;
            x.hl[base + k] = x.neg[c * x.N + k], x.tl[base + k] = -1, x.rsl[base + k] = 0.0f;
            if (k == 0) x.rowp[g] = base;
        }
    }
}

// One wave per chunk: the first list row of every group that has a positive in the chunk, in the
// order of the groups' first positives (glist[c * C + i], i < gcount[c]).
__global__ __launch_bounds__(64) void tneg_chunk_groups_kernel(NegIdx x, int32_t *glist, int32_t *gcount)
{
    const int64_t c = blockIdx.x;
    const int lane = threadIdx.x;
    int count = 0;
    for (int64_t i0 = 0; i0 < x.C; i0 += kWave) {
        const int64_t i = i0 + lane;
        const int64_t b = c * x.C + (i < x.C ? i : x.C - 1);
        const int g = x.k_inv[b];
        const bool rep = i < x.C && x.k_perm[x.k_seg[g]] == (int32_t)b;  // the stable sort puts the smallest b first
        const uint64_t m = __ballot(rep);
        if (rep) glist[c * x.C + count + __popcll(m & ((1ull << lane) - 1))] = x.rowp[g];
        count += __popcll(m);
    }
    if (lane == 0) gcount[c] = count;
}

// A row held by a wave: NQ float4 per lane (NQ = ceil(dim / 256) <= 4, a template parameter of
// the kernels so that narrow rows issue no idle loads).
template <int NQ>
struct NegRow {
    float4 v[NQ];
};

template <int NQ>
__device__ __forceinline__ NegRow<NQ> neg_load_row(const float *p, int d, int lane)
{
    NegRow<NQ> r;
#pragma unroll
    for (int q = 0; q < NQ; ++q) {
        const int j = q * 256 + lane * 4;
        const float4 v = *reinterpret_cast<const float4 *>(p + (j < d ? j : 0));  // clamped: unconditional load
        r.v[q] = j < d ? v : make_float4(0.f, 0.f, 0.f, 0.f);
    }
    return r;
}

template <int NQ>
__device__ __forceinline__ void neg_store_row(float *p, int d, int lane, const NegRow<NQ> &r)
{
#pragma unroll
    for (int q = 0; q < NQ; ++q) {
        const int j = q * 256 + lane * 4;
        if (j < d) *reinterpret_cast<float4 *>(p + j) = r.v[q];
    }
}

template <int P, int NQ>
__device__ __forceinline__ float neg_norm_partial(const NegRow<NQ> &a, const NegRow<NQ> &p)
{
    float s = 0.0f;
#pragma unroll
    for (int q = 0; q < NQ; ++q) {
        const float u0 = a.v[q].x - p.v[q].x, u1 = a.v[q].y - p.v[q].y, u2 = a.v[q].z - p.v[q].z, u3 = a.v[q].w - p.v[q].w;
        if constexpr (P == 1) s += (fabsf(u0) + fabsf(u1)) + (fabsf(u2) + fabsf(u3));
        else s = fmaf(u0, u0, fmaf(u1, u1, fmaf(u2, u2, fmaf(u3, u3, s))));
    }
    return s;
}

// acc += coef * phi(a - p), phi = sign (L1) or identity (L2: coef already carries 1 / norm)
template <int P, int NQ>
__device__ __forceinline__ void neg_accumulate(NegRow<NQ> &acc, const NegRow<NQ> &a, const NegRow<NQ> &p, float coef)
{
#pragma unroll
    for (int q = 0; q < NQ; ++q) {
        const float u0 = a.v[q].x - p.v[q].x, u1 = a.v[q].y - p.v[q].y, u2 = a.v[q].z - p.v[q].z, u3 = a.v[q].w - p.v[q].w;
        acc.v[q].x = fmaf(coef, P == 1 ? sgn(u0) : u0, acc.v[q].x);
        acc.v[q].y = fmaf(coef, P == 1 ? sgn(u1) : u1, acc.v[q].y);
        acc.v[q].z = fmaf(coef, P == 1 ? sgn(u2) : u2, acc.v[q].z);
        acc.v[q].w = fmaf(coef, P == 1 ? sgn(u3) : u3, acc.v[q].w);
    }
}

struct NegPairArgs {
    const float *ent;
    const float *y;         // projected list rows [L, d]
    float *pos, *neg;       // forward outputs (pos nullable)
    float *resid;           // forward: positives' residual rows [B, d] (nullable)
    const float *dpos, *dneg, *spos, *sneg;  // backward inputs (dpos / dneg nullable)
    float *xl, *ql, *qr;    // backward: left operands / upstream rows of the list, per-positive relation rows
};

// One wave per positive: pos[b] = ||y_pos||, neg[b][k] = ||a_b - P_(g(b),k)||.
template <int P, int NQ>
__global__ __launch_bounds__(256) void tneg_pair_fwd_kernel(NegIdx x, NegPairArgs a)
{
    const int lane = threadIdx.x & 63;
    const int64_t b = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (b >= x.B) return;
    const int d = x.d;
    const int N = (int)x.N;
    const NegRow<NQ> ya = neg_load_row<NQ>(a.y + (int64_t)x.rowa[b] * d, d, lane);
    const float *pg = a.y + (int64_t)x.rowp[x.k_inv[b]] * d;
    if (a.pos || a.resid) {
        const NegRow<NQ> yp = neg_load_row<NQ>(a.y + (int64_t)x.rowpos[b] * d, d, lane);
        NegRow<NQ> z;
#pragma unroll
        for (int q = 0; q < NQ; ++q) z.v[q] = make_float4(0.f, 0.f, 0.f, 0.f);
        const float s = wave_sum(neg_norm_partial<P, NQ>(yp, z));
        if (a.pos && lane == 0) a.pos[b] = P == 2 ? sqrtf(s) : s;
        if (a.resid) neg_store_row(a.resid + b * (int64_t)d, d, lane, yp);
    }
    for (int k0 = 0; k0 < N; k0 += 4) {  // four rows in flight
        NegRow<NQ> p[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) p[u] = neg_load_row<NQ>(pg + (int64_t)(k0 + u < N ? k0 + u : N - 1) * d, d, lane);
        float s[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) s[u] = neg_norm_partial<P, NQ>(ya, p[u]);
#pragma unroll
        for (int o = 32; o > 0; o >>= 1)
#pragma unroll
            for (int u = 0; u < 4; ++u) s[u] += __shfl_xor(s[u], o, kWave);
        if (lane < 4 && k0 + lane < N) {
            const float v = lane == 0 ? s[0] : (lane == 1 ? s[1] : (lane == 2 ? s[2] : s[3]));
            a.neg[b * (int64_t)N + k0 + lane] = P == 2 ? sqrtf(v) : v;
        }
    }
}

// Backward, one wave per positive: upstream rows of its two list rows (the positive's own residual
// row and its a row), their left operands, and the row that goes to the relation table.
template <int P, int NQ>
__global__ __launch_bounds__(256) void tneg_pair_bwd_a_kernel(NegIdx x, NegPairArgs a)
{
    const int lane = threadIdx.x & 63;
    const int64_t b = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (b >= x.B) return;
    const int d = x.d;
    const int N = (int)x.N;
    const int ra = x.rowa[b], rp = x.rowpos[b];
    const NegRow<NQ> ya = neg_load_row<NQ>(a.y + (int64_t)ra * d, d, lane);
    const float *pg = a.y + (int64_t)x.rowp[x.k_inv[b]] * d;
    NegRow<NQ> ga, z;
#pragma unroll
    for (int q = 0; q < NQ; ++q) ga.v[q] = make_float4(0.f, 0.f, 0.f, 0.f), z.v[q] = ga.v[q];
    if (a.dneg) {
        for (int k0 = 0; k0 < N; k0 += 4) {
            NegRow<NQ> p[4];
            float coef[4];
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                const int k = k0 + u < N ? k0 + u : N - 1;
                p[u] = neg_load_row<NQ>(pg + (int64_t)k * d, d, lane);
                const float g = a.dneg[b * (int64_t)N + k];
                float c = g;
                if constexpr (P == 2) {
                    const float s = a.sneg[b * (int64_t)N + k];
                    c = s > 0.0f ? g / s : 0.0f;
                }
                coef[u] = k0 + u < N ? c : 0.0f;
            }
#pragma unroll
            for (int u = 0; u < 4; ++u) neg_accumulate<P, NQ>(ga, ya, p[u], coef[u]);
        }
    }
    // the positive's own residual row
    const NegRow<NQ> yp = neg_load_row<NQ>(a.y + (int64_t)rp * d, d, lane);
    float gs = a.dpos ? a.dpos[b] : 0.0f;
    if constexpr (P == 2) {
        const float s = a.spos[b];
        gs = s > 0.0f ? gs / s : 0.0f;
    }
    NegRow<NQ> qp;
#pragma unroll
    for (int q = 0; q < NQ; ++q) qp.v[q] = make_float4(0.f, 0.f, 0.f, 0.f);
    neg_accumulate<P, NQ>(qp, yp, z, gs);
    const NegRow<NQ> eh = neg_load_row<NQ>(a.ent + x.h[b] * (int64_t)d, d, lane), et = neg_load_row<NQ>(a.ent + x.t[b] * (int64_t)d, d, lane);
    NegRow<NQ> xp, qr;
    const float sg = x.head ? -1.0f : 1.0f;
#pragma unroll
    for (int q = 0; q < NQ; ++q) {
        xp.v[q] = make_float4(eh.v[q].x - et.v[q].x, eh.v[q].y - et.v[q].y, eh.v[q].z - et.v[q].z, eh.v[q].w - et.v[q].w);
        qr.v[q] = make_float4(fmaf(sg, ga.v[q].x, qp.v[q].x), fmaf(sg, ga.v[q].y, qp.v[q].y), fmaf(sg, ga.v[q].z, qp.v[q].z),
                              fmaf(sg, ga.v[q].w, qp.v[q].w));
    }
    neg_store_row(a.ql + (int64_t)rp * d, d, lane, qp);
    neg_store_row(a.xl + (int64_t)rp * d, d, lane, xp);
    neg_store_row(a.ql + (int64_t)ra * d, d, lane, ga);
    neg_store_row(a.xl + (int64_t)ra * d, d, lane, x.head ? et : eh);
    neg_store_row(a.qr + b * (int64_t)d, d, lane, qr);
}

// Backward, upstream rows of the P rows: Q_(g,k) = - sum over the positives b of group g of their pair
// gradients.  The positives sit next to each other in the key order, so this is a segmented sum
// over the sorted positions whose terms are formed on the fly.  Level 1: a wave owns kNegSeg
// consecutive sorted positions and one negative k and walks them in order; a group that lies
// wholly inside the block is final, one that began in an earlier block goes to partial slot 0 of
// the block, one that continues past it to slot 1 (the scheme of seg_reduce.hip).  Level 2: the
// block in which a long group starts adds its slot-1 partial and the slot-0 partials of the
// following blocks.  Work is spread over B N / kNegSeg waves whatever the group sizes are (a hot
// relation's group has hundreds of positives); the order of the sum is fixed by the sorted order.
template <int P, int NQ>
__global__ __launch_bounds__(256) void tneg_pair_bwd_p1_kernel(NegIdx x, NegPairArgs a, const int32_t *k_sseg, float *partial)
{
    const int lane = threadIdx.x & 63;
    const int64_t w = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    const int N = (int)x.N, d = x.d;
    const int64_t j = w / N;
    const int k = (int)(w % N);
    const int64_t p0 = j * kNegSeg;
    if (p0 >= x.B) return;
    const int cnt = (int)(x.B - p0 < kNegSeg ? x.B - p0 : kNegSeg);
    int bb[kNegSeg], gg[kNegSeg];
#pragma unroll
    for (int q = 0; q < kNegSeg; ++q) {
        const int64_t pc = p0 + (q < cnt ? q : cnt - 1);  // clamped: unconditional loads, masked at their use
        bb[q] = x.k_perm[pc], gg[q] = k_sseg[pc];
    }
    const int g_before = p0 > 0 ? k_sseg[p0 - 1] : -1, g_after = p0 + cnt < x.B ? k_sseg[p0 + cnt] : -1;
    NegRow<NQ> acc;
#pragma unroll
    for (int e = 0; e < NQ; ++e) acc.v[e] = make_float4(0.f, 0.f, 0.f, 0.f);
    auto flush = [&](int g) {
        float *dst;
        if (g == g_before) dst = partial + ((j * N + k) * 2 + 0) * (int64_t)d;
        else if (g == g_after) dst = partial + ((j * N + k) * 2 + 1) * (int64_t)d;
        else dst = a.ql + (int64_t)(x.rowp[g] + k) * d;
        neg_store_row(dst, d, lane, acc);
    };
    constexpr int kFly = NQ == 1 ? 8 : (NQ == 2 ? 4 : 2);  // positions whose rows are in flight together
#pragma unroll
    for (int q0 = 0; q0 < kNegSeg; q0 += kFly) {
        NegRow<NQ> ya[kFly], pr[kFly];
        float coef[kFly];
#pragma unroll
        for (int u = 0; u < kFly; ++u) {
            const int q = q0 + u;
            ya[u] = neg_load_row<NQ>(a.y + (int64_t)x.rowa[bb[q]] * d, d, lane);
            pr[u] = neg_load_row<NQ>(a.y + (int64_t)(x.rowp[gg[q]] + k) * d, d, lane);
            float c = 0.0f;
            if (a.dneg) {  // uniform
                c = a.dneg[bb[q] * (int64_t)N + k];
                if constexpr (P == 2) {
                    const float sc = a.sneg[bb[q] * (int64_t)N + k];
                    c = sc > 0.0f ? c / sc : 0.0f;
                }
            }
            coef[u] = -c;
        }
#pragma unroll
        for (int u = 0; u < kFly; ++u) {
            const int q = q0 + u;
            if (q < cnt) {
                if (q > 0 && gg[q] != gg[q - 1]) {
                    flush(gg[q - 1]);
#pragma unroll
                    for (int e = 0; e < NQ; ++e) acc.v[e] = make_float4(0.f, 0.f, 0.f, 0.f);
                }
                neg_accumulate<P, NQ>(acc, ya[u], pr[u], coef[u]);
            }
        }
    }
    flush(gg[cnt - 1]);
}

template <int NQ>
__global__ __launch_bounds__(256) void tneg_pair_bwd_p2_kernel(NegIdx x, const int32_t *k_sseg, const float *partial, float *ql)
{
    const int lane = threadIdx.x & 63;
    const int64_t w = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    const int N = (int)x.N, d = x.d;
    const int64_t j = w / N;
    const int k = (int)(w % N);
    const int64_t p0 = j * kNegSeg;
    if (p0 >= x.B) return;
    const int64_t p1 = p0 + kNegSeg < x.B ? p0 + kNegSeg : x.B;
    const int g = k_sseg[p1 - 1];
    const int s0 = x.k_seg[g], s1 = x.k_seg[g + 1];
    if (s1 <= p0 + kNegSeg || s0 < p0) return;  // no group starts here and continues
    const int64_t je = (s1 - 1) / kNegSeg;
    NegRow<NQ> acc = neg_load_row<NQ>(partial + ((j * N + k) * 2 + 1) * (int64_t)d, d, lane);
    constexpr int kFly = NQ == 1 ? 8 : (NQ == 2 ? 4 : 2);
    for (int64_t jj = j + 1; jj <= je; jj += kFly) {
        NegRow<NQ> t[kFly];
#pragma unroll
        for (int u = 0; u < kFly; ++u) t[u] = neg_load_row<NQ>(partial + (((jj + u <= je ? jj + u : je) * N + k) * 2) * (int64_t)d, d, lane);
#pragma unroll
        for (int u = 0; u < kFly; ++u)
            if (jj + u <= je) {
#pragma unroll
                for (int e = 0; e < NQ; ++e)
                    acc.v[e] = make_float4(acc.v[e].x + t[u].v[e].x, acc.v[e].y + t[u].v[e].y, acc.v[e].z + t[u].v[e].z,
                                           acc.v[e].w + t[u].v[e].w);
            }
    }
    neg_store_row(ql + (int64_t)(x.rowp[g] + k) * d, d, lane, acc);
}

// Left operands of the P rows for dM: the negatives' entity rows in list order (one wave per row).
template <int NQ>
__global__ __launch_bounds__(256) void tneg_prow_operands_kernel(NegIdx x, const float *ent, float *xl)
{
    const int lane = threadIdx.x & 63;
    const int64_t w = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    const int64_t g = w / x.N;
    if (g >= x.k_num[0]) return;
    const int row = x.rowp[g] + (int)(w % x.N);
    neg_store_row(xl + (int64_t)row * x.d, x.d, lane, neg_load_row<NQ>(ent + x.hl[row] * (int64_t)x.d, x.d, lane));
}

// Occurrence rows in the order of the entity inspection, concat(h, t, neg): the list's dX rows are
// added up per positive (own row and a row: one wave each, workgroups [0, ceil(B / 4))) and per
// (chunk, negative) over the chunk's groups (one workgroup each: its four waves take the groups
// i = wave, wave + 4, ... and their sums are added in wave order through LDS).
template <int NQ>
__global__ __launch_bounds__(256) void tneg_occ_kernel(NegIdx x, const float *dxl, const int32_t *glist,
                                                       const int32_t *gcount, float *occ)
{
    __shared__ float4 s_part[3][NQ * kWave];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int d = x.d;
    const int64_t pos_blocks = ceil_div(x.B, 4);
    if ((int64_t)blockIdx.x < pos_blocks) {
        const int64_t w = (int64_t)blockIdx.x * 4 + wave;
        if (w >= x.B) return;
        const NegRow<NQ> dp = neg_load_row<NQ>(dxl + (int64_t)x.rowpos[w] * d, d, lane), da = neg_load_row<NQ>(dxl + (int64_t)x.rowa[w] * d, d, lane);
        NegRow<NQ> oh, ot;
#pragma unroll
        for (int q = 0; q < NQ; ++q) {
            const float4 p = dp.v[q], v = da.v[q];
            if (x.head) {
                oh.v[q] = p;
                ot.v[q] = make_float4(v.x - p.x, v.y - p.y, v.z - p.z, v.w - p.w);
            } else {
                oh.v[q] = make_float4(p.x + v.x, p.y + v.y, p.z + v.z, p.w + v.w);
                ot.v[q] = make_float4(-p.x, -p.y, -p.z, -p.w);
            }
        }
        neg_store_row(occ + w * (int64_t)d, d, lane, oh);
        neg_store_row(occ + (x.B + w) * (int64_t)d, d, lane, ot);
        return;
    }
    const int64_t q = (int64_t)blockIdx.x - pos_blocks;  // (chunk, negative); uniform for the workgroup
    if (q >= x.n_chunks * x.N) return;
    const int64_t c = q / x.N;
    const int k = (int)(q % x.N);
    const int cnt = gcount[c];
    NegRow<NQ> acc;
#pragma unroll
    for (int e = 0; e < NQ; ++e) acc.v[e] = make_float4(0.f, 0.f, 0.f, 0.f);
    constexpr int kFly = NQ == 1 ? 8 : (NQ == 2 ? 4 : 2);  // groups in flight per wave
    for (int i = wave; i < cnt; i += 4 * kFly) {
        NegRow<NQ> r[kFly];
#pragma unroll
        for (int u = 0; u < kFly; ++u) {
            const int iu = i + 4 * u;
            r[u] = neg_load_row<NQ>(dxl + (int64_t)(glist[c * x.C + (iu < cnt ? iu : i)] + k) * d, d, lane);
        }
#pragma unroll
        for (int u = 0; u < kFly; ++u)
            if (i + 4 * u < cnt) {
#pragma unroll
                for (int e = 0; e < NQ; ++e)
                    acc.v[e] = make_float4(acc.v[e].x + r[u].v[e].x, acc.v[e].y + r[u].v[e].y, acc.v[e].z + r[u].v[e].z,
                                           acc.v[e].w + r[u].v[e].w);
            }
    }
    if (wave > 0) {
#pragma unroll
        for (int e = 0; e < NQ; ++e) s_part[wave - 1][e * kWave + lane] = acc.v[e];
    }
    __syncthreads();
    if (wave == 0) {
#pragma unroll
        for (int e = 0; e < NQ; ++e) {
            const float4 p1 = s_part[0][e * kWave + lane], p2 = s_part[1][e * kWave + lane], p3 = s_part[2][e * kWave + lane];
            acc.v[e] = make_float4((acc.v[e].x + p1.x) + (p2.x + p3.x), (acc.v[e].y + p1.y) + (p2.y + p3.y),
                                   (acc.v[e].z + p1.z) + (p2.z + p3.z), (acc.v[e].w + p1.w) + (p2.w + p3.w));
        }
        neg_store_row(occ + (2 * x.B + q) * (int64_t)d, d, lane, acc);
    }
}

// ---- host side --------------------------------------------------------------------------------
// launch `stmt` with NQ_ = float4 per lane of a row (dim <= 1024: 1..4)
#define TNEG_BY_WIDTH(d_, stmt)            \
    do {                                   \
        const int nq_ = ((d_) + 255) / 256; \
        if (nq_ <= 1) {                    \
            constexpr int NQ_ = 1;         \
            stmt;                          \
        } else if (nq_ == 2) {             \
            constexpr int NQ_ = 2;         \
            stmt;                          \
        } else if (nq_ == 3) {             \
            constexpr int NQ_ = 3;         \
            stmt;                          \
        } else {                           \
            constexpr int NQ_ = 4;         \
            stmt;                          \
        }                                  \
    } while (0)
#define TNEG_BY_NORM(p_, kern, grid_, ...)                                                          \
    do {                                                                                            \
        if ((p_) == 1) hipLaunchKernelGGL((kern<1, NQ_>), grid_, dim3(256), 0, st, __VA_ARGS__);    \
        else hipLaunchKernelGGL((kern<2, NQ_>), grid_, dim3(256), 0, st, __VA_ARGS__);              \
    } while (0)
// The workspaces are sized for the worst case G = min(B, n_rel * n_chunks) groups (the count is only known on
// the device): about four arrays of (2 B + G N) * dim floats, with many relations about four times the
// B * N * dim floats of the flattened triples.  Above this many bytes (forward + backward) the path declines and
// the caller scores the flattened triples (or sees the shape in the error), instead of running out of memory.
constexpr size_t kNegWorkspaceCap = size_t(24) << 30;

static bool transr_neg_path_ok(const kge_tables *tab, const kge_batch *bat)
{
    if (tab->model != KGE_TRANSR || !bat->neg || !bat->rel_insp) return false;
    if (!mfma_path_ok(tab, bat) || gemm_lds_bytes((int)tab->dim) > kMaxGemmLds) return false;
    const NegShape s = neg_shape(tab, bat);
    if (!(s.n_chunks > 0 && tab->n_rel * s.n_chunks < (int64_t(1) << 31) && s.L_cap < (int64_t(1) << 31) &&
          s.L_cap * s.d < (int64_t(1) << 36)))
        return false;
    return neg_fwd_layout(tab, s).total + neg_bwd_layout(s).total <= kNegWorkspaceCap;
}

size_t transr_neg_fwd_workspace(const kge_tables *tab, const kge_batch *bat)
{
    if (!transr_neg_path_ok(tab, bat)) return 0;
    return neg_fwd_layout(tab, neg_shape(tab, bat)).total;
}

size_t transr_neg_bwd_workspace(const kge_tables *tab, const kge_batch *bat)
{
    if (!transr_neg_path_ok(tab, bat)) return 0;
    return neg_bwd_layout(neg_shape(tab, bat)).total;
}

static NegIdx neg_idx(const kge_tables *tab, const kge_batch *bat, const NegShape &s, const NegFwdLayout &l, char *ws)
{
    const kge_inspection *ri = bat->rel_insp;
    NegIdx x{};
    x.h = bat->h, x.r = bat->r, x.t = bat->t, x.neg = bat->neg;
    x.r_num = ri->num_unique, x.r_seg = ri->seg_offsets, x.r_perm = ri->perm, x.r_inv = ri->inverse, x.r_sseg = ri->sorted_seg;
    x.r_uniq = ri->unique_ids;
    x.keys = reinterpret_cast<int64_t *>(ws + l.keys);
    x.k_num = reinterpret_cast<int32_t *>(ws + l.knum);
    x.k_uniq = reinterpret_cast<int64_t *>(ws + l.kuniq);
    x.k_seg = reinterpret_cast<int32_t *>(ws + l.kseg);
    x.k_perm = reinterpret_cast<int32_t *>(ws + l.kperm);
    x.k_inv = reinterpret_cast<int32_t *>(ws + l.kinv);
    x.gstart = reinterpret_cast<int32_t *>(ws + l.gstart);
    x.segl = reinterpret_cast<int32_t *>(ws + l.segl);
    x.rowpos = reinterpret_cast<int32_t *>(ws + l.rowpos);
    x.rowa = reinterpret_cast<int32_t *>(ws + l.rowa);
    x.rowp = reinterpret_cast<int32_t *>(ws + l.rowp);
    x.hl = reinterpret_cast<int64_t *>(ws + l.hl);
    x.tl = reinterpret_cast<int64_t *>(ws + l.tl);
    x.rsl = reinterpret_cast<float *>(ws + l.rsl);
    x.B = s.B, x.N = s.N, x.C = s.C, x.n_chunks = s.n_chunks, x.G_cap = s.G_cap;
    x.d = (int)tab->dim, x.head = bat->neg_mode == KGE_NEG_HEAD ? 1 : 0;
    return x;
}

int launch_transr_neg_fwd(const kge_tables *tab, const kge_batch *bat, float *pos, float *neg, float *resid, void *workspace,
                          size_t workspace_bytes, hipStream_t st)
{
    if (!transr_neg_path_ok(tab, bat)) return KGE_EUNSUPPORTED;
    if (bat->fuse_inspection) return KGE_EINVAL;  // this path runs its own group inspection
    if (!neg) return KGE_EINVAL;
    const NegShape s = neg_shape(tab, bat);
    const NegFwdLayout l = neg_fwd_layout(tab, s);
    if (!workspace || workspace_bytes < l.total || !aligned16(workspace)) return KGE_EWORKSPACE;
    char *ws = static_cast<char *>(workspace);
    const NegIdx x = neg_idx(tab, bat, s, l, ws);
    const kge_inspection *ri = bat->rel_insp;
    const int d = (int)tab->dim;

    // groups: inspection of the keys relation * n_chunks + chunk
    hipLaunchKernelGGL(tneg_keys_kernel, dim3((unsigned)ceil_div(s.B, 256)), dim3(256), 0, st, x);
    const kge_inspection kin{s.B, tab->n_rel * s.n_chunks, const_cast<int32_t *>(x.k_num), const_cast<int64_t *>(x.k_uniq),
                             const_cast<int32_t *>(x.k_seg), const_cast<int32_t *>(x.k_perm), const_cast<int32_t *>(x.k_inv),
                             reinterpret_cast<int32_t *>(ws + l.ksseg)};
    const int64_t *parts[1] = {x.keys};
    const int64_t lens[1] = {s.B};
    if (const int rc = kge_inspect(parts, lens, 1, kin.n_rows, &kin, ws + l.kws, l.kws_bytes, st)) return rc;
    timeline_mark(bat->timeline, st, "inspect(relation, chunk)");

    // the list and its tile plans
    hipLaunchKernelGGL(tneg_gstart_kernel, dim3((unsigned)ceil_div(s.U_cap + 1, 256)), dim3(256), 0, st, x);
    const int64_t list_threads = s.B + s.G_cap * s.N;
    const int64_t list_blocks = ceil_div(list_threads, 256);
    hipLaunchKernelGGL(tneg_list_kernel, dim3((unsigned)(list_blocks < 8192 ? list_blocks : 8192)), dim3(256), 0, st, x);
    TilePlan plan = plan_at(ws + l.plan, s.tiles, 0), dplan = dplan_at(ws + l.dplan, s.dtiles, s.dsplit, d);
    hipLaunchKernelGGL(transr_plan_kernel, dim3(2), dim3(1024), 0, st, ri->num_unique, x.segl, ri->unique_ids, plan, kTM, dplan,
                       kDmChunk, dm_nib(d), dm_small_max(d));
    timeline_mark(bat->timeline, st, "row list + transr_plan_kernel");

    // one grouped pass projects every list row
    float *y = reinterpret_cast<float *>(ws + l.y);
    GemmArgs ga{tab->ent, tab->rel, tab->aux, x.hl, nullptr, x.tl, nullptr, x.segl, ri->num_unique, ri->unique_ids,
                plan, nullptr, x.rsl, nullptr, y, nullptr, nullptr, d, tab->norm_p, (int)s.U_cap, (int)s.tiles, BwdSrc{}};
    const size_t lds = gemm_lds_bytes(d);
    if (const int rc = allow_lds<3>(lds)) return rc;
    hipLaunchKernelGGL(transr_gemm_kernel<3>, dim3((unsigned)(s.tiles + s.U_cap)), dim3(256), lds, st, ga, FusedInsp{});
    timeline_mark(bat->timeline, st, "transr_gemm_kernel<list>");

    NegPairArgs pa{};
    pa.ent = tab->ent, pa.y = y, pa.pos = pos, pa.neg = neg, pa.resid = resid;
    const dim3 pgrid((unsigned)ceil_div(s.B, 4));
    TNEG_BY_WIDTH(d, TNEG_BY_NORM(tab->norm_p, tneg_pair_fwd_kernel, pgrid, x, pa));
    timeline_mark(bat->timeline, st, "tneg_pair_fwd_kernel");
    KGE_CHECK_LAUNCH();
    return KGE_OK;
}

int launch_transr_neg_bwd(const kge_tables *tab, const kge_batch *bat, const kge_saved *saved, const float *dpos,
                          const float *dneg, const kge_grads *grads, void *workspace, size_t workspace_bytes, hipStream_t st)
{
    if (!transr_neg_path_ok(tab, bat)) return KGE_EUNSUPPORTED;
    if (bat->fuse_inspection) return KGE_EINVAL;
    const NegShape s = neg_shape(tab, bat);
    const NegFwdLayout fl = neg_fwd_layout(tab, s);
    const NegBwdLayout l = neg_bwd_layout(s);
    // the forward call's workspace holds the groups, the list, the plans and the projected rows
    if (!saved->fwd_workspace || saved->fwd_workspace_bytes < fl.total) return KGE_EINVAL;
    if (!workspace || workspace_bytes < l.total || !aligned16(workspace)) return KGE_EWORKSPACE;
    if (!grads->ent_rows || !grads->rel_rows || !grads->aux_rows) return KGE_EINVAL;
    // the per-positive kernel reads the positive scores whenever the norm is L2 (dpos == NULL stands for
    // zeros, not for "skip"), so they are required as in launch_transr_bwd
    if (tab->norm_p == 2 && (!saved->pos || (dneg && !saved->neg))) return KGE_EINVAL;
    if (!bat->ent_insp || bat->ent_insp->n != 2 * s.B + s.NN) return KGE_ESHAPE;
    char *fws = static_cast<char *>(const_cast<void *>(saved->fwd_workspace)), *ws = static_cast<char *>(workspace);
    const NegIdx x = neg_idx(tab, bat, s, fl, fws);
    const kge_inspection *ri = bat->rel_insp;
    const int d = (int)tab->dim;
    float *y = reinterpret_cast<float *>(fws + fl.y);
    float *xl = reinterpret_cast<float *>(ws + l.xl), *ql = reinterpret_cast<float *>(ws + l.ql);
    float *dxl = reinterpret_cast<float *>(ws + l.dxl), *occ = reinterpret_cast<float *>(ws + l.occ);
    float *qr = reinterpret_cast<float *>(ws + l.qr);
    int32_t *glist = reinterpret_cast<int32_t *>(ws + l.glist), *gcount = reinterpret_cast<int32_t *>(ws + l.gcount);
    TilePlan plan = plan_at(fws + fl.plan, s.tiles, 0), dplan = dplan_at(fws + fl.dplan, s.dtiles, s.dsplit, d);

    NegPairArgs pa{};
    pa.ent = tab->ent, pa.y = y, pa.dpos = dpos, pa.dneg = dneg, pa.spos = saved->pos, pa.sneg = saved->neg;
    pa.xl = xl, pa.ql = ql, pa.qr = qr;
    const dim3 agrid((unsigned)ceil_div(s.B, 4)), pgrid((unsigned)ceil_div(s.G_cap * s.N, 4));
    TNEG_BY_WIDTH(d, TNEG_BY_NORM(tab->norm_p, tneg_pair_bwd_a_kernel, agrid, x, pa));
    float *ppart = reinterpret_cast<float *>(ws + l.ppart);
    const int32_t *k_sseg = reinterpret_cast<const int32_t *>(fws + fl.ksseg);
    const dim3 sgrid((unsigned)ceil_div(ceil_div(s.B, kNegSeg) * s.N, 4));
    TNEG_BY_WIDTH(d, TNEG_BY_NORM(tab->norm_p, tneg_pair_bwd_p1_kernel, sgrid, x, pa, k_sseg, ppart));
    TNEG_BY_WIDTH(d, hipLaunchKernelGGL(tneg_pair_bwd_p2_kernel<NQ_>, sgrid, dim3(256), 0, st, x, k_sseg, ppart, ql));
    TNEG_BY_WIDTH(d, hipLaunchKernelGGL(tneg_prow_operands_kernel<NQ_>, pgrid, dim3(256), 0, st, x, tab->ent, xl));
    hipLaunchKernelGGL(tneg_chunk_groups_kernel, dim3((unsigned)s.n_chunks), dim3(64), 0, st, x, glist, gcount);
    timeline_mark(bat->timeline, st, "tneg_pair_bwd kernels");

    // dX = Q M^T over the list (rows stay in list order), dM = X^T Q per relation
    GemmArgs ga{tab->ent, tab->rel, tab->aux, x.hl, nullptr, x.tl, nullptr, x.segl, ri->num_unique, ri->unique_ids,
                plan, ql, nullptr, nullptr, nullptr, dxl, nullptr, d, tab->norm_p, (int)s.U_cap, (int)s.tiles, BwdSrc{}};
    const size_t lds = gemm_lds_bytes(d);
    if (const int rc = allow_lds<2>(lds)) return rc;
    hipLaunchKernelGGL(transr_gemm_kernel<2>, dim3((unsigned)(s.tiles + s.U_cap)), dim3(256), lds, st, ga, FusedInsp{});
    timeline_mark(bat->timeline, st, "transr_gemm_kernel<dX>");
    DmArgs da{xl, ql, x.segl, dplan, grads->aux_rows, reinterpret_cast<float *>(ws + l.dpart), d, ri->num_unique,
              BwdSrc{}, nullptr, nullptr, 0};
    hipLaunchKernelGGL(transr_dm_kernel, dim3((unsigned)kDmWgs), dim3(256), dm_lds_bytes(d), st, da, FusedInsp{}, SegL1Rider{});
    timeline_mark(bat->timeline, st, "transr_dm_kernel");
    TNEG_BY_WIDTH(d, hipLaunchKernelGGL(tneg_occ_kernel<NQ_>, dim3((unsigned)(ceil_div(s.B, 4) + s.NN)), dim3(256), 0, st, x, dxl,
                                        glist, gcount, occ));
    timeline_mark(bat->timeline, st, "tneg_occ_kernel");
    KGE_CHECK_LAUNCH();
    if (bat->insp_ready && hipStreamWaitEvent(st, reinterpret_cast<hipEvent_t>(bat->insp_ready), 0) != hipSuccess)
        return KGE_ELAUNCH;
    const SegJob jobs[2] = {{occ, bat->ent_insp, d, grads->ent_rows, reinterpret_cast<float *>(ws + l.part_e), false},
                            {qr, ri, d, grads->rel_rows, reinterpret_cast<float *>(ws + l.part_r), false}};
    const SumRider finish = dm_finish_rider(da, s.dsplit);  // the split groups' partial matrices
    return launch_seg_reduce_jobs(jobs, 2, st, bat->timeline, &finish);
}
