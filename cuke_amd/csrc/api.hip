// extern "C" entry points: argument validation and kernel dispatch.
#include <stdlib.h>

#include "inspector_mid.hpp"

namespace kge {
int launch_score_pos(const kge_tables *, const kge_batch *, float *, float *, float *, hipStream_t);
int launch_score_pos_fused(const kge_tables *, const kge_batch *, float *, float *, float *, const FusedInsp *,
                           hipStream_t);
int launch_score_neg(const kge_tables *, const kge_batch *, const float *, const float *, float *, float *,
                     const FusedInsp *, void *, size_t, hipStream_t, float *carry_pos);
bool score_neg_carries_positives(const kge_tables *, const kge_batch *);
size_t neg_split_workspace(const kge_tables *, const kge_batch *);
int launch_transr_fwd(const kge_tables *, const kge_batch *, float *, float *, void *, size_t, hipStream_t);
bool back_rows_ok(const kge_tables *, const kge_batch *);
int launch_rescal_head_rows(const kge_tables *, const kge_batch *, float *, void *, size_t, hipStream_t);
size_t transr_fwd_workspace(const kge_tables *, const kge_batch *);
int launch_transr_plan(const kge_tables *, const kge_batch *, void *, size_t, hipStream_t);
int launch_transr_neg_fwd(const kge_tables *, const kge_batch *, float *, float *, float *, void *, size_t, hipStream_t);
size_t transr_neg_fwd_workspace(const kge_tables *, const kge_batch *);

__global__ void check_indices_kernel(const int64_t *idx, int64_t n, int64_t n_rows, int32_t *flag)
{
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) {
        const int64_t v = idx[i];
        if (v < 0 || v >= n_rows) *flag = 1;  // benign race: every writer stores 1
    }
}

__global__ void flatten_negatives_kernel(const int64_t *h, const int64_t *r, const int64_t *t, const int64_t *neg,
                                         int64_t B, int64_t C, int64_t N, int head, int64_t *hf, int64_t *rf,
                                         int64_t *tf)
{
    const int64_t total = B * (1 + N);
    for (int64_t p = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; p < total; p += (int64_t)gridDim.x * blockDim.x) {
        if (p < B) {
            hf[p] = h[p], rf[p] = r[p], tf[p] = t[p];
        } else {
            const int64_t q = p - B, b = q / N, k = q % N;
            const int64_t e = neg[(b / C) * N + k];
            hf[p] = head ? e : h[b], rf[p] = r[b], tf[p] = head ? t[b] : e;
        }
    }
}

__device__ __forceinline__ uint64_t splitmix64(uint64_t z)
{
    z += 0x9E3779B97F4A7C15ull;
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    return z ^ (z >> 31);
}

__global__ void sample_negatives_kernel(int64_t *out, int64_t count, uint64_t n_ent, uint64_t seed, uint64_t step)
{
    const uint64_t base = seed ^ splitmix64(step);
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < count; i += (int64_t)gridDim.x * blockDim.x) {
        const uint64_t x = splitmix64(base ^ ((uint64_t)i * 0x9E3779B97F4A7C15ull));
        out[i] = (int64_t)__umul64hi(x, n_ent);  // uniform over [0, n_ent)
    }
}

static int validate_tables(const kge_tables *tab)
{
    if (!tab || !tab->ent) return KGE_EINVAL;
    if (tab->model < KGE_TRANSE || tab->model > KGE_RESCAL) return KGE_EINVAL;
    if (tab->dim <= 0 || tab->dim > (1 << 20) || tab->n_ent <= 0) return KGE_ESHAPE;
    const bool complex_rows = tab->model == KGE_COMPLEX || tab->model == KGE_ROTATE;
    if (complex_rows && (tab->dim & 1)) return KGE_ESHAPE;
    if (tab->rel_dim != rel_width(tab->model, tab->dim)) return KGE_ESHAPE;
    if (tab->rel_dim > 0 && (!tab->rel || tab->n_rel <= 0)) return KGE_EINVAL;
    if (aux_width(tab->model, tab->dim) > 0 && !tab->aux) return KGE_EINVAL;
    if (tab->flags & ~KGE_PAIR_SUMS_VALU) return KGE_EINVAL;
    const bool normed = tab->model == KGE_TRANSE || tab->model == KGE_TRANSH || tab->model == KGE_TRANSR;
    if (normed && tab->norm_p != 1 && tab->norm_p != 2) return KGE_EINVAL;
    return KGE_OK;
}

static int validate_batch(const kge_batch *bat)
{
    if (!bat || bat->batch < 0) return KGE_EINVAL;
    if (bat->batch > 0 && (!bat->h || !bat->r || !bat->t)) return KGE_EINVAL;
    if (bat->batch >= (int64_t(1) << 31)) return KGE_ESHAPE;
    if (bat->neg) {
        if (bat->chunk <= 0 || bat->n_neg <= 0) return KGE_ESHAPE;
        if (bat->batch % bat->chunk != 0) return KGE_ESHAPE;
        if (bat->neg_mode != KGE_NEG_TAIL && bat->neg_mode != KGE_NEG_HEAD) return KGE_EINVAL;
    }
    return KGE_OK;
}
}  // namespace kge

using namespace kge;

extern "C" {

const char *kge_strerror(int status)
{
    switch (status) {
    case KGE_OK: return "ok";
    case KGE_EINVAL: return "invalid argument (null pointer, unknown model or norm order)";
    case KGE_ESHAPE: return "inconsistent sizes (batch % chunk, odd complex dim, bad rel_dim)";
    case KGE_ELAUNCH: return "kernel launch failed";
    case KGE_EWORKSPACE: return "workspace missing or too small";
    case KGE_EUNSUPPORTED: return "combination not supported";
    default: return "unknown status";
    }
}

int kge_abi_version(void) { return 7; }

int kge_back_rows_ok(const kge_tables *tab, const kge_batch *bat)
{
    if (!tab || !bat || bat->batch <= 0 || validate_tables(tab) != KGE_OK) return 0;
    return kge::back_rows_ok(tab, bat) ? 1 : 0;
}

kge_timeline *kge_timeline_create(int32_t capacity)
{
    if (capacity <= 0 || capacity > 4096) return nullptr;
    kge_timeline *tl = static_cast<kge_timeline *>(calloc(1, sizeof(kge_timeline)));
    if (!tl) return nullptr;
    tl->events = static_cast<void **>(calloc((size_t)capacity, sizeof(void *)));
    tl->labels = static_cast<const char **>(calloc((size_t)capacity, sizeof(char *)));
    tl->capacity = capacity;
    bool ok = tl->events && tl->labels;
    hipEvent_t ev;
    if (ok && hipEventCreate(&ev) == hipSuccess) tl->begin = ev;
    else ok = false;
    for (int i = 0; ok && i < capacity; ++i) {
        if (hipEventCreate(&ev) == hipSuccess) tl->events[i] = ev;
        else ok = false;
    }
    if (!ok) {
        kge_timeline_destroy(tl);
        return nullptr;
    }
    return tl;
}

void kge_timeline_destroy(kge_timeline *tl)
{
    if (!tl) return;
    if (tl->begin) (void)hipEventDestroy(reinterpret_cast<hipEvent_t>(tl->begin));
    for (int i = 0; tl->events && i < tl->capacity; ++i)
        if (tl->events[i]) (void)hipEventDestroy(reinterpret_cast<hipEvent_t>(tl->events[i]));
    free(tl->events);
    free(const_cast<char **>(tl->labels));
    free(tl);
}

int kge_timeline_begin(kge_timeline *tl, void *stream)
{
    if (!tl || !tl->begin) return KGE_EINVAL;
    tl->count = 0, tl->dropped = 0;
    return hipEventRecord(reinterpret_cast<hipEvent_t>(tl->begin), as_stream(stream)) == hipSuccess ? KGE_OK : KGE_ELAUNCH;
}

int kge_timeline_mark(kge_timeline *tl, const char *label, void *stream)
{
    if (!tl || !label) return KGE_EINVAL;
    if (tl->count >= tl->capacity) return KGE_EWORKSPACE;
    const int before = tl->count;
    timeline_mark(tl, as_stream(stream), label);
    return tl->count == before + 1 ? KGE_OK : KGE_ELAUNCH;
}

int kge_timeline_elapsed(const kge_timeline *tl, float *ms)
{
    if (!tl || !ms || !tl->begin) return KGE_EINVAL;
    if (tl->dropped > 0) return KGE_EWORKSPACE;  // more kernels than capacity (or a failed record): no truncated table
    hipEvent_t prev = reinterpret_cast<hipEvent_t>(tl->begin);
    for (int i = 0; i < tl->count; ++i) {
        hipEvent_t cur = reinterpret_cast<hipEvent_t>(tl->events[i]);
        if (hipEventElapsedTime(&ms[i], prev, cur) != hipSuccess) return KGE_ELAUNCH;
        prev = cur;
    }
    return tl->count;
}

size_t kge_score_fwd_workspace(const kge_tables *tab, const kge_batch *bat)
{
    if (!tab || !bat || bat->batch < 0) return 0;
    if (tab->model == KGE_TRANSR && bat->neg && bat->rel_insp) {  // shared negatives: group list + projected rows
        const size_t nb = transr_neg_fwd_workspace(tab, bat);
        if (nb) return nb;
    }
    if ((tab->model == KGE_TRANSR || tab->model == KGE_RESCAL) && bat->rel_insp) return transr_fwd_workspace(tab, bat);
    if (tab->model == KGE_TRANSE || tab->model == KGE_ROTATE) return neg_split_workspace(tab, bat);  // small batches only
    return 0;
}

int kge_transr_plan(const kge_tables *tab, const kge_batch *bat, void *workspace, size_t workspace_bytes, void *stream)
{
    int rc = validate_tables(tab);
    if (rc) return rc;
    if ((rc = validate_batch(bat))) return rc;
    if ((tab->model != KGE_TRANSR && tab->model != KGE_RESCAL) || !bat->rel_insp) return KGE_EINVAL;
    KGE_CLEAR_LAUNCH_ERRORS();
    return launch_transr_plan(tab, bat, workspace, workspace_bytes, as_stream(stream));
}

int kge_residual_fwd(const kge_tables *tab, const kge_batch *bat, float *out, void *workspace,
                     size_t workspace_bytes, void *stream)
{
    int rc = validate_tables(tab);
    if (rc) return rc;
    if ((rc = validate_batch(bat))) return rc;
    if (!out && bat->batch > 0) return KGE_EINVAL;
    if (tab->model != KGE_TRANSE && tab->model != KGE_TRANSH && tab->model != KGE_TRANSR)
        return KGE_EUNSUPPORTED;  // the other models have scalar outputs only
    KGE_CLEAR_LAUNCH_ERRORS();
    if (tab->model == KGE_TRANSR && bat->rel_insp)
        return launch_transr_fwd(tab, bat, nullptr, out, workspace, workspace_bytes, as_stream(stream));
    return launch_score_pos(tab, bat, nullptr, out, nullptr, as_stream(stream));
}

int kge_score_fwd(const kge_tables *tab, const kge_batch *bat, float *pos, float *neg,
                  float *side_pos, float *side_neg, float *residual, void *workspace, size_t workspace_bytes,
                  void *stream)
{
    int rc = validate_tables(tab);
    if (rc) return rc;
    if ((rc = validate_batch(bat))) return rc;
    hipStream_t st = as_stream(stream);
    KGE_CLEAR_LAUNCH_ERRORS();
    const bool want_neg = neg && bat->neg;
    if (bat->back_rows && !back_rows_ok(tab, bat)) return KGE_EUNSUPPORTED;  // (only TransR's grouped forward writes them)
    if (want_neg && (tab->model == KGE_TRANSH || tab->model == KGE_TRANSF) && !side_pos) return KGE_EINVAL;
    if (want_neg && tab->model == KGE_ROTATE && !residual) return KGE_EINVAL;  // rotated heads buffer
    if (want_neg && tab->model == KGE_RESCAL && !residual) return KGE_EINVAL;  // the projected rows are the pair kernel's queries
    const bool rescal_head = want_neg && tab->model == KGE_RESCAL && bat->neg_mode == KGE_NEG_HEAD;
    if (rescal_head && !bat->rel_insp) return KGE_EUNSUPPORTED;  // (the rows Proj[r] E[t] come from the grouped pass)
    // fused inspection: first digit pass with the per-positive kernel, second with the tile kernel
    const bool grouped_model = tab->model == KGE_TRANSR || tab->model == KGE_RESCAL;
    const bool fuse = bat->fuse_inspection != 0 && !grouped_model;  // (the grouped kernels plan their own riders)
    if (bat->fuse_inspection && grouped_model && !(bat->rel_insp && (pos || residual))) return KGE_EINVAL;
    FusedInsp fi0{}, fi1{};
    if (fuse) {
        if (!want_neg || !bat->insp_jobs || !(pos || side_pos || residual) || bat->batch == 0) return KGE_EINVAL;
        if ((rc = plan_fused_inspection(bat->insp_jobs, 2, 0, &fi0))) return rc;
        if ((rc = plan_fused_inspection(bat->insp_jobs, 2, 1, &fi1))) return rc;
    }
    if (want_neg && tab->model == KGE_TRANSR && bat->rel_insp)  // positives and shared negatives in one grouped pass
        return launch_transr_neg_fwd(tab, bat, pos, neg, residual, workspace, workspace_bytes, st);
    // TransE, DistMult / ComplEx on the matrix-core tiles: the positives ride in the tile launch where
    // nothing else does (score_neg_carries_positives; also with the reduction axis of small TransE
    // batches split, where their workgroups follow tile_blocks * ksplit tile workgroups).  `pos` is then
    // written by the negatives' launch, and its timeline entry "score_neg_kernel" includes the positives.
    const bool carry = want_neg && pos && !side_pos && !residual && !fuse && score_neg_carries_positives(tab, bat);
    if (!carry && (pos || side_pos || residual)) {
        if (rescal_head) {
            // corrupted heads: the positives' scores from the usual pass, then `residual` takes the rows
            // u_b = Proj[r_b] E[t_b] that the pair scores E[h'] . u_b (and the backward pass) are formed from
            rc = pos ? launch_transr_fwd(tab, bat, pos, nullptr, workspace, workspace_bytes, st)
                     : launch_transr_plan(tab, bat, workspace, workspace_bytes, st);
            if (!rc) rc = launch_rescal_head_rows(tab, bat, residual, workspace, workspace_bytes, st);
        } else if ((tab->model == KGE_TRANSR || tab->model == KGE_RESCAL) && bat->rel_insp)
            rc = launch_transr_fwd(tab, bat, pos, residual, workspace, workspace_bytes, st);
        else {
            rc = launch_score_pos_fused(tab, bat, pos, residual, side_pos, fuse ? &fi0 : nullptr, st);
            timeline_mark(bat->timeline, st, "score_pos_kernel");
        }
        if (rc) return rc;
    }
    if (want_neg) {
        rc = launch_score_neg(tab, bat, side_pos, (tab->model == KGE_ROTATE || tab->model == KGE_RESCAL) ? residual : nullptr, neg, side_neg,
                              fuse ? &fi1 : nullptr, workspace, workspace_bytes, st, carry ? pos : nullptr);
        timeline_mark(bat->timeline, st, "score_neg_kernel");
        return rc;
    }
    return KGE_OK;
}

int kge_flatten_negatives(const kge_batch *bat, int64_t *h_flat, int64_t *r_flat, int64_t *t_flat, void *stream)
{
    const int rc = validate_batch(bat);
    if (rc) return rc;
    if (!bat->neg) return KGE_EINVAL;
    if (bat->batch == 0) return KGE_OK;
    if (!h_flat || !r_flat || !t_flat) return KGE_EINVAL;
    const int64_t total = bat->batch * (1 + bat->n_neg);
    if (total >= (int64_t(1) << 31)) return KGE_ESHAPE;
    const int64_t blocks = ceil_div(total, 256);
    hipLaunchKernelGGL(flatten_negatives_kernel, dim3((unsigned)(blocks < 4096 ? blocks : 4096)), dim3(256), 0,
                       as_stream(stream), bat->h, bat->r, bat->t, bat->neg, bat->batch, bat->chunk, bat->n_neg,
                       bat->neg_mode == KGE_NEG_HEAD ? 1 : 0, h_flat, r_flat, t_flat);
    KGE_CHECK_LAUNCH();
    return KGE_OK;
}

int kge_sample_negatives(int64_t *out, int64_t count, int64_t n_ent, uint64_t seed, uint64_t step, void *stream)
{
    if (count < 0 || n_ent <= 0) return KGE_ESHAPE;
    if (count == 0) return KGE_OK;
    if (!out) return KGE_EINVAL;
    const int64_t blocks = ceil_div(count, 256);
    hipLaunchKernelGGL(sample_negatives_kernel, dim3((unsigned)(blocks < 2048 ? blocks : 2048)), dim3(256), 0,
                       as_stream(stream), out, count, (uint64_t)n_ent, seed, step);
    KGE_CHECK_LAUNCH();
    return KGE_OK;
}

int kge_check_indices(const int64_t *idx, int64_t n, int64_t n_rows, int32_t *flag, void *stream)
{
    if (!flag || (n > 0 && !idx) || n < 0) return KGE_EINVAL;
    if (n == 0) return KGE_OK;
    hipLaunchKernelGGL(check_indices_kernel, dim3((unsigned)ceil_div(n, 256)), dim3(256), 0,
                       as_stream(stream), idx, n, n_rows, flag);
    KGE_CHECK_LAUNCH();
    return KGE_OK;
}

}  // extern "C"
