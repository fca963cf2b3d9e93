// TransR / RESCAL with a row width that is not a multiple of four.
//
// The grouped kernels move everything in 128-bit pieces: entity rows, the rows of the projections that
// stream past as matrix-core operands, the gradient matrices.  A row width d with d % 4 != 0 leaves none of
// those rows 16-byte aligned.  Instead of a second, scalar-load form of every grouped kernel, such a batch is
// copied into a compact, padded problem in the caller's workspace -- the 2 B entity rows of the batch, the
// relation rows and the projections of the relation groups that occur, each padded with zeros to
// dp = 4 * ceil(d / 4) columns (and rows) -- and the grouped kernels run on that: zero columns add exact
// zeros to every sum.  Results are copied back without the padding.  It costs one more pass over the
// projections that the batch uses (read d x d, write dp x dp) per call; the reference's transR() has no
// restriction on dim at all (apps/kge/kge.py:321-343), so the shapes have to work, at whatever speed.
//
// Compact ids: entity row b of the padded table is E[h[b]], row B + b is E[t[b]]; relation group g of the
// inspection is relation g of the padded tables (unique_ids replaced by 0, 1, 2, ...).
//
// This file is included by transr.hip (inside namespace kge) below the grouped kernels.

static int64_t pad4(int64_t d) { return (d + 3) & ~int64_t(3); }

static bool pad_path_ok(const kge_tables *tab, const kge_batch *bat)
{
    return (tab->model == KGE_TRANSR || tab->model == KGE_RESCAL) && bat->rel_insp && !bat->neg && tab->dim % 4 != 0 &&
           pad4(tab->dim) <= kMaxDimMfma && bat->rel_insp->n == bat->batch && bat->batch > 0 &&
           gemm_lds_bytes((int)pad4(tab->dim)) <= kMaxGemmLds;
}

struct PadLayout {
    size_t inner, ep, rp, pp, hp, tp, uid, residp, ent_rows, rel_rows, aux_rows, total;
    int64_t B, d, dp, G;
};

struct PadCtx {
    kge_tables tab;
    kge_batch bat;
    kge_inspection ri;
};

// the padded problem's descriptors (pointers into the workspace `ws` laid out by `l`)
static void pad_ctx(const kge_tables *tab, const kge_batch *bat, const PadLayout &l, char *ws, PadCtx *c)
{
    c->tab = *tab;
    c->tab.dim = l.dp;
    c->tab.rel_dim = tab->model == KGE_TRANSR ? l.dp : 0;
    c->tab.n_ent = 2 * l.B;
    c->tab.n_rel = l.G;
    c->tab.ent = reinterpret_cast<float *>(ws + l.ep);
    c->tab.rel = tab->model == KGE_TRANSR ? reinterpret_cast<float *>(ws + l.rp) : nullptr;
    c->tab.aux = reinterpret_cast<float *>(ws + l.pp);
    c->ri = *bat->rel_insp;
    c->ri.unique_ids = reinterpret_cast<int64_t *>(ws + l.uid);
    c->ri.n_rows = l.G;
    c->bat = *bat;
    c->bat.h = reinterpret_cast<int64_t *>(ws + l.hp);
    c->bat.t = reinterpret_cast<int64_t *>(ws + l.tp);
    c->bat.rel_insp = &c->ri;
    c->bat.fuse_inspection = 0;
    c->bat.insp_jobs = nullptr;
}

// `bwd`: also the padded gradient arrays and the inner backward workspace (else the inner forward workspace)
static PadLayout pad_layout(const kge_tables *tab, const kge_batch *bat, bool bwd)
{
    PadLayout l{};
    l.B = bat->batch, l.d = tab->dim, l.dp = pad4(tab->dim);
    l.G = l.B < tab->n_rel ? l.B : tab->n_rel;
    size_t o = 0;
    auto take = [&](size_t bytes) {
        const size_t at = o;
        o += up256(bytes > 0 ? bytes : 1);
        return at;
    };
    // sizes of the inner workspaces only depend on the shapes: descriptors without pointers are enough
    kge_tables t2 = *tab;
    t2.dim = l.dp, t2.rel_dim = tab->model == KGE_TRANSR ? l.dp : 0, t2.n_ent = 2 * l.B, t2.n_rel = l.G;
    kge_batch b2 = *bat;
    b2.neg = nullptr;
    l.inner = take(bwd ? make_rplan(&t2, &b2).total : transr_fwd_workspace(&t2, &b2));
    l.ep = take(sizeof(float) * (size_t)(2 * l.B * l.dp));
    l.rp = take(tab->model == KGE_TRANSR ? sizeof(float) * (size_t)(l.G * l.dp) : 0);
    l.pp = take(sizeof(float) * (size_t)(l.G * l.dp * l.dp));
    l.hp = take(sizeof(int64_t) * (size_t)l.B);
    l.tp = take(sizeof(int64_t) * (size_t)l.B);
    l.uid = take(sizeof(int64_t) * (size_t)l.G);
    l.residp = take(sizeof(float) * (size_t)(l.B * l.dp));
    if (bwd) {
        l.ent_rows = take(sizeof(float) * (size_t)(2 * l.B * l.dp));
        l.rel_rows = take(tab->model == KGE_TRANSR ? sizeof(float) * (size_t)(l.G * l.dp) : 0);
        l.aux_rows = take(sizeof(float) * (size_t)(l.G * l.dp * l.dp));
    }
    l.total = o;
    return l;
}

// Entity rows of the batch and the compact index arrays.
__global__ void pad_entities_kernel(const float *ent, const int64_t *h, const int64_t *t, int64_t B, int d, int dp, float *ep,
                                    int64_t *hp, int64_t *tp)
{
    const int64_t total = 2 * B * dp;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (int64_t)gridDim.x * blockDim.x) {
        const int64_t row = i / dp;
        const int j = (int)(i % dp);
        const int64_t id = row < B ? h[row] : t[row - B];
        ep[i] = j < d ? ent[id * d + j] : 0.0f;
        if (j == 0) {
            if (row < B) hp[row] = row;
            else tp[row - B] = row;
        }
    }
}

// Relation rows and projections of the groups that occur (group g -> relation g of the padded tables).
// `only_ids`: just the compact relation ids (all a tile plan needs).
__global__ void pad_relations_kernel(const float *rel, const float *proj, const int32_t *num_unique, const int64_t *unique_ids, int d,
                                     int dp, float *rp, float *pp, int64_t *uid, int only_ids)
{
    const int U = num_unique[0];
    const int64_t stride = (int64_t)gridDim.x * blockDim.x, first = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    for (int64_t g = first; g < U; g += stride) uid[g] = g;
    if (only_ids) return;
    if (rp)
        for (int64_t i = first; i < (int64_t)U * dp; i += stride) {
            const int64_t g = i / dp;
            const int j = (int)(i % dp);
            rp[i] = j < d ? rel[unique_ids[g] * d + j] : 0.0f;
        }
    const int64_t dd = (int64_t)dp * dp;
    for (int64_t i = first; i < (int64_t)U * dd; i += stride) {
        const int64_t g = i / dd;
        const int r = (int)((i % dd) / dp), j = (int)(i % dp);
        pp[i] = (r < d && j < d) ? proj[unique_ids[g] * (int64_t)d * d + (int64_t)r * d + j] : 0.0f;
    }
}

// [n, rows, cols] out of an array with padded pitches: dst[i][r][j] = src[i][r][j], r < rows, j < cols.
// n comes from the device (count[0], at most n_cap) or, with count == null, is n_cap.
__global__ void unpad_kernel(const float *src, float *dst, const int32_t *count, int64_t n_cap, int rows, int cols, int src_rows,
                             int src_cols)
{
    int64_t n = count ? count[0] : n_cap;
    n = n < n_cap ? n : n_cap;
    const int64_t per = (int64_t)rows * cols, total = n * per;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (int64_t)gridDim.x * blockDim.x) {
        const int64_t m = i / per;
        const int r = (int)((i % per) / cols), j = (int)(i % cols);
        dst[i] = src[(m * src_rows + r) * (int64_t)src_cols + j];
    }
}

// one row of `cols` floats per item into rows of pitch `dp`, zero beyond cols (the residual rows for backward)
__global__ void pad_rows_kernel(const float *src, float *dst, int64_t n, int cols, int dp)
{
    const int64_t total = n * dp;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (int64_t)gridDim.x * blockDim.x) {
        const int j = (int)(i % dp);
        dst[i] = j < cols ? src[(i / dp) * cols + j] : 0.0f;
    }
}

static unsigned pad_grid(int64_t items) { const int64_t b = ceil_div(items > 0 ? items : 1, 256); return (unsigned)(b < 4096 ? b : 4096); }

static void launch_pad_tables(const kge_tables *tab, const kge_batch *bat, const PadLayout &l, char *ws, hipStream_t st)
{
    const kge_inspection *ri = bat->rel_insp;
    hipLaunchKernelGGL(pad_entities_kernel, dim3(pad_grid(2 * l.B * l.dp)), dim3(256), 0, st, tab->ent, bat->h, bat->t, l.B, (int)l.d,
                       (int)l.dp, reinterpret_cast<float *>(ws + l.ep), reinterpret_cast<int64_t *>(ws + l.hp),
                       reinterpret_cast<int64_t *>(ws + l.tp));
    hipLaunchKernelGGL(pad_relations_kernel, dim3(pad_grid(l.G * l.dp * l.dp)), dim3(256), 0, st, tab->rel, tab->aux, ri->num_unique,
                       ri->unique_ids, (int)l.d, (int)l.dp, tab->model == KGE_TRANSR ? reinterpret_cast<float *>(ws + l.rp) : nullptr,
                       reinterpret_cast<float *>(ws + l.pp), reinterpret_cast<int64_t *>(ws + l.uid), 0);
}

static size_t transr_fwd_workspace_padded(const kge_tables *tab, const kge_batch *bat) { return pad_layout(tab, bat, false).total; }
static size_t transr_bwd_workspace_padded(const kge_tables *tab, const kge_batch *bat) { return pad_layout(tab, bat, true).total; }

static int launch_transr_plan_padded(const kge_tables *tab, const kge_batch *bat, void *workspace, size_t workspace_bytes, hipStream_t st)
{
    const PadLayout l = pad_layout(tab, bat, false);
    if (!workspace || workspace_bytes < l.total || !aligned16(workspace)) return KGE_EWORKSPACE;
    char *ws = static_cast<char *>(workspace);
    PadCtx c;
    pad_ctx(tab, bat, l, ws, &c);
    const kge_inspection *ri = bat->rel_insp;
    hipLaunchKernelGGL(pad_relations_kernel, dim3(pad_grid(l.G)), dim3(256), 0, st, nullptr, nullptr, ri->num_unique, ri->unique_ids,
                       (int)l.d, (int)l.dp, nullptr, nullptr, reinterpret_cast<int64_t *>(ws + l.uid), 1);
    return launch_transr_plan(&c.tab, &c.bat, ws + l.inner, l.ep - l.inner, st);
}

static int launch_transr_fwd_padded(const kge_tables *tab, const kge_batch *bat, float *pos, float *resid, void *workspace,
                                    size_t workspace_bytes, hipStream_t st)
{
    if (bat->fuse_inspection) return KGE_EINVAL;  // (no riding inspection on the padded path)
    const PadLayout l = pad_layout(tab, bat, false);
    if (!workspace || workspace_bytes < l.total || !aligned16(workspace)) return KGE_EWORKSPACE;
    char *ws = static_cast<char *>(workspace);
    PadCtx c;
    pad_ctx(tab, bat, l, ws, &c);
    launch_pad_tables(tab, bat, l, ws, st);
    float *residp = reinterpret_cast<float *>(ws + l.residp);
    const int rc = launch_transr_fwd(&c.tab, &c.bat, pos, resid ? residp : nullptr, ws + l.inner, l.ep - l.inner, st);
    if (rc) return rc;
    if (resid)
        hipLaunchKernelGGL(unpad_kernel, dim3(pad_grid(l.B * l.d)), dim3(256), 0, st, residp, resid, nullptr, l.B, 1, (int)l.d, 1,
                           (int)l.dp);
    KGE_CHECK_LAUNCH();
    return KGE_OK;
}

static int launch_transr_bwd_padded(const kge_tables *tab, const kge_batch *bat, const kge_saved *saved, const float *dpos,
                                    const kge_grads *grads, void *workspace, size_t workspace_bytes, hipStream_t st)
{
    const bool rescal = tab->model == KGE_RESCAL;
    if (bat->fuse_inspection) return KGE_EINVAL;
    if (grads->aux_factor_max != 0) return KGE_EUNSUPPORTED;  // (factored gradients: row widths that are multiples of four)
    if (!saved->residual || !grads->aux_rows || !grads->ent_rows || (!rescal && !grads->rel_rows)) return KGE_EINVAL;
    if (!rescal && tab->norm_p == 2 && !saved->pos) return KGE_EINVAL;
    const PadLayout l = pad_layout(tab, bat, true);
    if (!workspace || workspace_bytes < l.total || !aligned16(workspace)) return KGE_EWORKSPACE;
    if (bat->ent_insp->n != 2 * bat->batch) return KGE_ESHAPE;
    char *ws = static_cast<char *>(workspace);
    PadCtx c;
    pad_ctx(tab, bat, l, ws, &c);
    launch_pad_tables(tab, bat, l, ws, st);
    float *residp = reinterpret_cast<float *>(ws + l.residp);
    hipLaunchKernelGGL(pad_rows_kernel, dim3(pad_grid(l.B * l.dp)), dim3(256), 0, st, saved->residual, residp, l.B, (int)l.d, (int)l.dp);
    kge_saved s2 = *saved;
    s2.residual = residp;
    s2.fwd_workspace = nullptr, s2.fwd_workspace_bytes = 0;  // (plans of its own: the caller's forward workspace has another layout)
    kge_grads g2{};
    g2.ent_rows = reinterpret_cast<float *>(ws + l.ent_rows);
    g2.rel_rows = rescal ? nullptr : reinterpret_cast<float *>(ws + l.rel_rows);
    g2.aux_rows = reinterpret_cast<float *>(ws + l.aux_rows);
    const int rc = launch_transr_bwd(&c.tab, &c.bat, &s2, dpos, &g2, ws + l.inner, l.ep - l.inner, st);
    if (rc) return rc;
    const kge_inspection *ri = bat->rel_insp;
    hipLaunchKernelGGL(unpad_kernel, dim3(pad_grid(2 * l.B * l.d)), dim3(256), 0, st, g2.ent_rows, grads->ent_rows, bat->ent_insp->num_unique,
                       2 * l.B, 1, (int)l.d, 1, (int)l.dp);
    if (!rescal)
        hipLaunchKernelGGL(unpad_kernel, dim3(pad_grid(l.G * l.d)), dim3(256), 0, st, g2.rel_rows, grads->rel_rows, ri->num_unique, l.G, 1,
                           (int)l.d, 1, (int)l.dp);
    hipLaunchKernelGGL(unpad_kernel, dim3(pad_grid(l.G * l.d * l.d)), dim3(256), 0, st, g2.aux_rows, grads->aux_rows, ri->num_unique, l.G,
                       (int)l.d, (int)l.d, (int)l.dp, (int)l.dp);
    KGE_CHECK_LAUNCH();
    return KGE_OK;
}
