// One step of a staged training loop in one call: host-side sequencing only, no kernels of its own.
//
// A step of the small benchmark shapes is 45 us of device work in eight kernel launches on two streams;
// issued call by call from Python (inspect, record, wait, forward, loss, backward, record) the host needs
// longer than that for the calls themselves, and the device waits.  kge_train_step_staged enqueues the same
// sequence -- the inspection of the NEXT batch on the side stream, the step of the CURRENT batch on the
// main stream, the events between the two -- from native code, so what remains on the host is the launches.
// The reference has no training loop; its one call per score function is replaced by this one call per step.
#include "common.hpp"

using namespace kge;

static hipEvent_t as_event(void *e) { return reinterpret_cast<hipEvent_t>(e); }

extern "C" int kge_train_step_staged(const kge_tables *tab, kge_step_batch *cur, kge_step_batch *next, const kge_step_buffers *buf,
                                     void *stream, void *side_stream)
{
    if (!tab || (!cur && !next) || (cur && !buf)) return KGE_EINVAL;
    hipStream_t st = as_stream(stream), side = as_stream(side_stream);
    const bool projection = tab->model == KGE_TRANSR || tab->model == KGE_RESCAL;
    if (next) {
        if (!next->inspected || !next->bat.insp_jobs) return KGE_EINVAL;
        const kge_inspect_job *jobs = next->bat.insp_jobs;
        // the step that read these inspection buffers last must have been enqueued AND finished
        if (next->released_valid && next->released && hipStreamWaitEvent(side, as_event(next->released), 0) != hipSuccess)
            return KGE_ELAUNCH;
        int rc = KGE_OK;
        if (projection && !next->bat.neg && next->fwd_workspace) {
            // the relation groups drive the forward pass: inspected and planned here, a step ahead
            if (!next->planned) return KGE_EINVAL;
            // (both index sets in one batch of launches, then the plans: the step waits for all of it at once)
            if ((rc = kge_inspect_batch(jobs, 2, side_stream))) return rc;
            if ((rc = kge_transr_plan(tab, &next->bat, next->fwd_workspace, next->fwd_workspace_bytes, side_stream))) return rc;
            if (hipEventRecord(as_event(next->planned), side) != hipSuccess) return KGE_ELAUNCH;
            next->bat.plans_ready = 1;
        } else if (projection) {
            rc = kge_inspect_batch(&jobs[0], 1, side_stream);  // (the relations are inspected on the main stream, by the step)
        } else {
            rc = kge_inspect_batch(jobs, 2, side_stream);
        }
        if (rc) return rc;
        if (hipEventRecord(as_event(next->inspected), side) != hipSuccess) return KGE_ELAUNCH;
    }
    if (!cur) return KGE_OK;
    if (!cur->inspected || !cur->released) return KGE_EINVAL;
    kge_batch *bat = &cur->bat;
    bat->fuse_inspection = 0;
    bat->insp_ready = cur->inspected;  // backward waits for it right before its segmented reduction
    void *fws = buf->fwd_workspace;
    size_t fws_bytes = buf->fwd_workspace_bytes;
    if (projection && !bat->neg && cur->fwd_workspace) {
        if (!bat->plans_ready || !cur->planned) return KGE_EINVAL;  // staged by an earlier call
        // plans and entity inspection were enqueued together, a step ahead: one wait on the later event covers both
        if (hipStreamWaitEvent(st, as_event(cur->inspected), 0) != hipSuccess) return KGE_ELAUNCH;
        bat->insp_ready = nullptr;
        fws = cur->fwd_workspace, fws_bytes = cur->fwd_workspace_bytes;
    } else if (projection) {
        const int rc = kge_inspect_batch(&bat->insp_jobs[1], 1, stream);
        if (rc) return rc;
    }
    int rc = kge_score_fwd(tab, bat, buf->pos, buf->neg, buf->side_pos, buf->side_neg, buf->residual, fws, fws_bytes, stream);
    if (rc) return rc;
    if (buf->loss) {
        if ((rc = kge_margin_loss(buf->pos, buf->neg, bat->batch, bat->n_neg, buf->margin, buf->sign, buf->loss, buf->dpos, buf->dneg,
                                  buf->loss_workspace, buf->loss_workspace_bytes, stream)))
            return rc;
    }
    kge_saved saved{buf->pos, buf->neg, buf->side_pos, buf->side_neg, buf->residual, nullptr, 0, bat->back_rows};
    if (projection) saved.fwd_workspace = fws, saved.fwd_workspace_bytes = fws_bytes;
    if ((rc = kge_score_bwd(tab, bat, &saved, buf->dpos, buf->dneg, &buf->grads, buf->bwd_workspace, buf->bwd_workspace_bytes, stream)))
        return rc;
    if (hipEventRecord(as_event(cur->released), st) != hipSuccess) return KGE_ELAUNCH;
    cur->released_valid = 1;
    return KGE_OK;
}
