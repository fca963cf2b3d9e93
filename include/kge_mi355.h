/*
 * kge_mi355 -- C ABI of the MI355X (gfx950) KGE score-function library.
 *
 * This is the boundary a host program binds instead of the reference's
 * JIT-loaded pybind11 modules:
 *   - pycuke1/run/gpu.py:4-20 + pycuke1/codegen/gpu_template.cu:8-17
 *       module.run(batch, dim, nnodes, Eemb, h, t, nedges, Remb, r, ...) -> Tensor
 *       (argument order per model: apps/kge/test_cuke.py:54,104,153,198,244)
 *   - apps/kge/inspection/inspector.cu:139-147
 *       gpu_sort(relation, r_Uniq, r_Buffer, uniq_cnt, batch, rel_num)
 *
 * Conventions
 *   - every pointer is DEVICE memory unless its comment says "host";
 *   - the library never allocates device memory: outputs and workspaces are
 *     caller-allocated, workspace sizes come from the *_workspace() calls;
 *   - `stream` is a hipStream_t passed as void*; calls only enqueue work and
 *     never synchronise;
 *   - return value: KGE_OK or a negative kge_status_t; kge_strerror() names it;
 *   - tables are fp32 row-major with 16-byte aligned base pointers; index
 *     arrays are int64 (the reference's GPU surface, pycuke1/codegen/gpu.py:200-201);
 *   - entity rows of ComplEx / RotatE are stored [re(dim/2) | im(dim/2)];
 *     RotatE relation rows are dim/2 phase angles.
 */
#ifndef KGE_MI355_H
#define KGE_MI355_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef enum kge_model_t {
    KGE_TRANSE = 0,   /* apps/kge/kge.py:273-293 */
    KGE_TRANSH = 1,   /* apps/kge/kge.py:296-318 */
    KGE_TRANSR = 2,   /* apps/kge/kge.py:321-343 */
    KGE_DISTMULT = 3, /* not in the reference: s = sum h*r*t */
    KGE_COMPLEX = 4,  /* not in the reference: s = Re<h, r, conj t> */
    KGE_ROTATE = 5,   /* not in the reference: s = gamma - sum |h e^{i theta} - t| */
    KGE_TRANSF = 6,   /* apps/kge/kge.py:346-366 */
    KGE_RESCAL = 7    /* apps/kge/kge.py:369-390 */
} kge_model_t;

typedef enum kge_status_t {
    KGE_OK = 0,
    KGE_EINVAL = -1,       /* null pointer, bad enum, bad norm order */
    KGE_ESHAPE = -2,       /* sizes inconsistent (batch % chunk, dim parity, alignment) */
    KGE_ELAUNCH = -3,      /* hipGetLastError() reported a failed launch */
    KGE_EWORKSPACE = -4,   /* workspace missing or too small */
    KGE_EUNSUPPORTED = -5  /* combination not implemented */
} kge_status_t;

/* Embedding tables of one model. */
typedef struct kge_tables {
    int32_t model;     /* kge_model_t */
    int32_t norm_p;    /* 1 or 2: norm of the TransE / TransH / TransR residual */
    float gamma;       /* RotatE offset */
    int32_t flags;     /* 0, or KGE_PAIR_SUMS_VALU */
    int64_t dim;       /* floats per entity row */
    int64_t rel_dim;   /* floats per relation row: dim, or dim/2 for RotatE, 0 for RESCAL */
    int64_t n_ent;
    int64_t n_rel;
    const float *ent;  /* [n_ent, dim]                               (Eemb) */
    const float *rel;  /* [n_rel, rel_dim]                           (Remb) */
    const float *aux;  /* TransH normals [n_rel, dim] (Pemb); TransR / RESCAL
                          projections [n_rel, dim, dim] (Proj); else NULL */
} kge_tables;

/* kge_tables.flags.  The shared-negative tile kernels of DistMult / ComplEx sum their pair
   products on the matrix cores (fp32 MFMA, fp32 accumulate) unless this bit asks for the vector
   ALUs; both forms meet the same tolerance.  The choice travels with the call, so concurrent
   callers cannot disturb each other.  No counterpart in the reference. */
enum { KGE_PAIR_SUMS_VALU = 1 };

/*
 * Optional per-kernel timeline of a call (kge_batch.timeline): after every kernel it launches,
 * kge_score_fwd / kge_score_bwd record events[count] on the call's stream, store the kernel's
 * name in labels[count] and advance count, until capacity is reached.  Kernel k's duration is
 * the time between events k-1 and k (`begin` for k = 0) once the stream has drained.
 * Host memory only; meant for measurement runs, not for the training loop.  No counterpart in
 * the reference.
 *   kge_timeline_create   allocates the struct and its events (hipEventCreate, timing enabled)
 *   kge_timeline_begin    count = 0 and records `begin` on the stream
 *   kge_timeline_mark     the caller's own entry (work enqueued between two library calls)
 *   kge_timeline_elapsed  ms[k] for k < count; call after the stream has been synchronised;
 *                         returns count or a negative status (KGE_EWORKSPACE when the call launched
 *                         more kernels than `capacity`, or an event could not be recorded: `dropped`
 *                         counts the entries that are missing, so a truncated table is never returned)
 */
typedef struct kge_timeline {
    void *begin;          /* hipEvent_t */
    void **events;        /* host array of `capacity` hipEvent_t */
    const char **labels;  /* host array of `capacity` slots, filled with static strings */
    int32_t capacity;
    int32_t count;        /* in / out */
    int32_t dropped;      /* entries lost since kge_timeline_begin (timeline full, failed event record) */
    int32_t reserved;
} kge_timeline;
kge_timeline *kge_timeline_create(int32_t capacity);
void kge_timeline_destroy(kge_timeline *tl);
int kge_timeline_begin(kge_timeline *tl, void *stream);
int kge_timeline_mark(kge_timeline *tl, const char *label, void *stream);
int kge_timeline_elapsed(const kge_timeline *tl, float *ms);

/*
 * Result of inspecting one index multiset (kge_inspect).  For idx[n]:
 *   unique_ids[0..U)   distinct ids, strictly ascending
 *   seg_offsets[0..U]  sorted positions where each id's run starts; [U] = n
 *   perm[n]            stable sort permutation: idx[perm[p]] ascending in p and
 *                      perm ascending inside a run
 *   inverse[n]         unique_ids[inverse[i]] == idx[i]
 *   sorted_seg[n]      inverse[perm[p]]: the run each sorted position belongs to
 *   num_unique[1]      U
 * Positions are int32 (n < 2^31); ids stay int64.
 */
typedef struct kge_inspection {
    int64_t n;
    int64_t n_rows;
    int32_t *num_unique;
    int64_t *unique_ids;   /* capacity n */
    int32_t *seg_offsets;  /* capacity n + 1 */
    int32_t *perm;         /* capacity n */
    int32_t *inverse;      /* capacity n */
    int32_t *sorted_seg;   /* capacity n */
} kge_inspection;

enum { KGE_NEG_TAIL = 0, KGE_NEG_HEAD = 1 };

/* One batch of triples.  neg == NULL: positives only. */
typedef struct kge_batch {
    int64_t batch;       /* B positives */
    const int64_t *h;    /* [B] head entity ids */
    const int64_t *r;    /* [B] relation ids */
    const int64_t *t;    /* [B] tail entity ids */
    const int64_t *neg;  /* [B / chunk * n_neg] shared negative entity ids, chunk-major */
    int64_t chunk;       /* positives per chunk; B % chunk == 0 */
    int64_t n_neg;       /* negatives per chunk: positive b is scored against
                            neg[(b / chunk) * n_neg + k], k < n_neg
                            (layout of apps/examples/examples.py:1404-1444) */
    /* inspection of concat(h, t, neg) (entity table) and of r (relation tables);
       needed by kge_score_bwd; rel_insp also by TransR forward */
    const kge_inspection *ent_insp;
    const kge_inspection *rel_insp;
    /* Optional hipEvent_t (as void*).  When set, the inspections may still be in flight on
       another stream: kge_score_bwd makes its stream wait on this event immediately before
       the first kernel that reads ent_insp (the segmented reduction), so the inspector runs
       concurrently with the forward pass and the gradient tile kernels.  rel_insp is NOT
       covered when the model is TransR / RESCAL (their forward already consumed it). */
    void *insp_ready;
    /* Which side of the positive the shared negatives replace: KGE_NEG_TAIL scores
       (h_b, r_b, neg_k), the layout of apps/examples/examples.py:1404-1444; KGE_NEG_HEAD scores
       (neg_k, r_b, t_b), the head-corrupted batches of apps/kge/data/sampler.py:287-353
       (neg_head).  Zero-initialised structs get KGE_NEG_TAIL. */
    int32_t neg_mode;
    /* Non-zero: the inspector's workgroups ride in front of the score kernels' own in the same
       launches, which takes the inspection off the critical path without a second stream.
       insp_jobs points to two jobs, [0] for the entity index set (concat(h, t, neg)) and [1] for r,
       whose `out` are the structs ent_insp / rel_insp point to.
       - Shared negatives (TransE, TransH, DistMult, ComplEx, RotatE): both jobs ride; histogram
         and first digit pass with the two forward kernels of kge_score_fwd (pos and neg scores
         must be requested), last pass and dedup with the two gradient kernels of kge_score_bwd.
       - TransR / RESCAL on their grouped path (no negatives, rel_insp complete before
         kge_score_fwd): job [0] rides with the forward GEMM, then (after one step in a launch of its
         own) with the dX and dM kernels of kge_score_bwd; job [1] is not used.
       Requirements: each riding index set at most 65536 ids, tables of at most 2^22 rows
       (kge_fused_inspection_ok says whether a batch qualifies); kge_score_fwd and kge_score_bwd
       must both be called, in this order, on one stream, and the riding inspections hold their
       result only after kge_score_bwd.  No counterpart in the reference, whose inspector is a
       separate call (apps/kge/kge.py:249-271). */
    int32_t fuse_inspection;
    const struct kge_inspect_job *insp_jobs;
    kge_timeline *timeline;  /* optional, see kge_timeline; NULL: nothing is recorded */
    /* TransR / RESCAL on their grouped path: non-zero = the workspace handed to kge_score_fwd already
       holds this batch's tile plans (kge_transr_plan ran on it after rel_insp was complete), so the
       forward call launches no plan kernel.  Lets a training loop inspect the relations and plan a
       batch ahead on another stream. */
    int32_t plans_ready;
    int32_t reserved;
    /* TransR on its grouped path without shared negatives, optional (kge_back_rows_ok says whether a batch
       qualifies; kge_score_fwd returns KGE_EUNSUPPORTED for a batch that sets it and does not): [B, dim]
       floats that kge_score_fwd fills with z_b = phi(y_b) Proj[r_b]^T, y_b the residual row of triple b and
       phi = sign for L1, identity for L2, formed by the forward kernel while it holds the projection.  The
       entity gradient of triple b is +-coef_b z_b (coef_b = dpos_b for L1, dpos_b / pos_b for L2), so a
       backward call that is handed the rows (kge_saved.back_rows) needs no second pass over the
       projections: it launches no dX kernel and its reduction scales the rows as it loads them.  The
       residual rows must be requested in the same call.  No counterpart in the reference, which has no
       executed backward pass (apps/kge/kge.py:393-515). */
    float *back_rows;
} kge_batch;

/* Forward outputs that backward consumes. */
typedef struct kge_saved {
    const float *pos;       /* [B] positive scores */
    const float *neg;       /* [B, n_neg] negative scores (NULL without negatives) */
    const float *side_pos;  /* [B]: TransH w.h per positive (w.t with KGE_NEG_HEAD); TransF with
                               negatives r.h (r.t); TransR: unused */
    const float *side_neg;  /* [2, B, n_neg]: TransH, plane 0 = w_b . e_k per pair (e_k the negative),
                               plane 1 = sum_i phi(u_i) w_i (phi = sign for L1, u/||u|| for L2) */
    const float *residual;  /* [B, dim]: TransR residual rows / RESCAL E[h] Proj[r] rows (with shared negatives
                               that replace the head: Proj[r] E[t] rows);
                               RotatE: rotated heads h e^{i theta} as [re | im]
                               (with KGE_NEG_HEAD: counter-rotated tails t e^{-i theta}) */
    /* TransR / RESCAL, optional: the workspace the forward call of this batch was given (it
       holds the tile plans of the relation groups); kge_score_bwd then reuses them instead of
       building its own.  NULL / 0: backward plans for itself.  Required for TransR with shared
       negatives (the group list and the projected rows live there). */
    const void *fwd_workspace;
    size_t fwd_workspace_bytes;
    /* TransR, optional: the rows kge_score_fwd wrote to kge_batch.back_rows for this batch (see there).
       NULL: kge_score_bwd forms the entity gradients with its own pass over the projections. */
    const float *back_rows;
} kge_saved;

/* Sparse row gradients: row u of each array belongs to the u-th unique id of the
 * matching inspection (ent_insp for ent_rows, rel_insp for rel_rows / aux_rows). */
typedef struct kge_grads {
    float *ent_rows;  /* [ent_insp->n, dim]        first U_ent rows written */
    float *rel_rows;  /* [B, rel_dim]              first U_rel rows written */
    float *aux_rows;  /* TransH: [B, dim]; TransR / RESCAL: [min(B, n_rel), dim*dim] */
    /* TransR / RESCAL without shared negatives, optional: FACTORED projection gradients of the small
       relation groups.  The gradient of relation group u (the u-th unique relation, sorted positions
       p in [seg_offsets[u], seg_offsets[u+1]) of rel_insp) is the sum over its triples of the outer
       products x_p^T q_p (x_p = E[h] - E[t], or E[h] for RESCAL; q_p the upstream row of the projected
       vector).  A group of one triple, as most relations of a long-tailed batch are, costs dim*dim
       floats of memory traffic to write out and again to read in the optimizer, for 2*dim floats of
       information.  With aux_factor_max = m in 1..4, a group of at most m triples leaves its rows
       x_p in aux_x[p] and q_p in aux_q[p] and its aux_rows[u] is NOT written; larger groups are written
       dense as always (their aux_x / aux_q rows are not written).  kge_sparse_sgd_factored /
       kge_sparse_adagrad_factored apply either form.  aux_factor_max = 0: every group dense (the
       form the parity tests check; the factored rows are tested against it).  No counterpart in the
       reference, whose printed gradient kernels are per-triple dense (apps/kge/kge.py:413-418). */
    float *aux_x;            /* [B, dim], 16-byte aligned */
    float *aux_q;            /* [B, dim], 16-byte aligned */
    int32_t aux_factor_max;  /* 0..4 */
    int32_t reserved;
} kge_grads;

const char *kge_strerror(int status);
int kge_abi_version(void);

/*
 * Residual vectors, the reference's output for TransE / TransH / TransR:
 *   out[b][:] = (E[h]-E[t]) + R[r]                       (kge.py:290)
 *             ... - (P[r].(E[h]-E[t])) P[r]              (kge.py:315)
 *             = (E[h]-E[t]) Proj[r] + R[r]               (kge.py:340)
 * Replaces module.run(...) of pycuke1/codegen/gpu_template.cu:8-13.
 * out: [B, dim].  TransE is bit-exact with the generated CPU loop.
 */
int kge_residual_fwd(const kge_tables *tab, const kge_batch *bat, float *out, void *workspace,
                     size_t workspace_bytes, void *stream);

/*
 * Scalar scores.  pos[B]; neg[B, n_neg] when bat->neg is set (either may be
 * NULL to skip).  side_pos / side_neg are optional save-for-backward outputs
 * (see kge_saved; required later by kge_score_bwd for TransH; side_pos is also required when
 * TransF scores shared negatives: the pair kernel reads r.h from it).
 * Scalar-score models of the reference: TransF / RESCAL (kge.py:363,387).
 * TransR / RESCAL: with bat->rel_insp (relation groups) the projection runs as grouped
 * per-relation MFMA contractions and needs kge_score_fwd_workspace() bytes of workspace;
 * without it every triple streams its own projection.  `residual` [B, dim] receives the
 * projected rows (TransR: the residual, RESCAL: E[h] Proj[r]) that kge_score_bwd consumes.
 * TransR with shared negatives (bat->neg, bat->rel_insp and neg all set; dim % 4 == 0, dim <= 1024):
 * the pair scores of the reference's neg_transR (apps/examples/examples.py:1447-1480, one
 * vector x matrix product per (positive, negative) pair) are formed from two projections,
 * (x - n) M + R = (x M + R) - n M, and every negative is projected once per (relation, chunk) group
 * of the batch instead of once per pair.  pos, neg and residual ([B, dim], the positives' residual
 * rows) come out of the one call; the workspace (kge_score_fwd_workspace with bat->neg set) keeps
 * the group list and the projected rows and must be handed to kge_score_bwd as
 * kge_saved.fwd_workspace.  TransR shapes outside the grouped kernels are scored through
 * kge_flatten_negatives.
 * RESCAL with shared negatives that replace the tail (KGE_NEG_TAIL): the pair score
 * (E[h] Proj[r]) . E[t'] needs no projection of the negatives, so pos, neg and `residual` ([B, dim],
 * the projected rows E[h] Proj[r], required) come out of one call: the grouped pass over the B
 * positives, then the dot-product tile kernel of DistMult with the projected rows as its query rows.
 * kge_score_bwd chains the pairs' gradient through the same B rows.  With KGE_NEG_HEAD the pair score is
 * E[h'] . (Proj[r] E[t]): `residual` then receives the rows Proj[r_b] E[t_b] (one more grouped pass, with the
 * transposed projections), which are the tile's query rows and what kge_score_bwd expects in kge_saved.residual.
 * TransE / RotatE with shared negatives on small batches (the 32 x 32 pair tiles would leave one or
 * two workgroups per CU): given kge_score_fwd_workspace() bytes of workspace the reduction axis of
 * every tile is split over up to four workgroups (partial score planes in the workspace, a finishing
 * kernel); without the workspace the same call runs one workgroup per tile.
 * TransE, and DistMult / ComplEx on the matrix-core tiles: when pos and neg are both requested, no
 * side output is and no inspection rides along, the positives are scored by extra workgroups of the
 * shared-negative launch (one launch instead of two; a timeline then has no "score_pos_kernel"
 * entry and its "score_neg_kernel" entry includes the positives).  Results are the same bits.
 * RotatE: `residual` [B, dim] receives the rotated heads h e^{i theta}; the shared-negative
 * kernels (forward and backward) load them instead of recomputing a sincos per element, so it
 * is required whenever negatives are scored (filled by this call when pos is requested, or
 * left from an earlier call on the same batch).
 */
size_t kge_score_fwd_workspace(const kge_tables *tab, const kge_batch *bat);
/* TransR / RESCAL without negatives: builds the tile plans of the relation groups (bat->rel_insp, complete
   on `stream`) into `workspace` (kge_score_fwd_workspace bytes), the part of kge_score_fwd that only
   depends on the relation ids.  Pass the same workspace to kge_score_fwd with bat->plans_ready set.
   No counterpart in the reference. */
int kge_transr_plan(const kge_tables *tab, const kge_batch *bat, void *workspace, size_t workspace_bytes,
                    void *stream);
int kge_score_fwd(const kge_tables *tab, const kge_batch *bat, float *pos, float *neg,
                  float *side_pos, float *side_neg, float *residual, void *workspace,
                  size_t workspace_bytes, void *stream);

/*
 * Index inspector: radix sort + dedup of up to four concatenated int64 index
 * arrays over a table of n_rows rows.  Stands where the reference calls
 * inspector() / gpu_sort (apps/kge/kge.py:249-271, inspector.cu:139-143); its
 * output is the full sorted/unique/segment structure rather than the
 * reference's per-16 cache slots (for those see kge_build_index).
 * parts / part_len are HOST arrays of n_parts device pointers / lengths.
 */
size_t kge_inspect_workspace(int64_t n, int64_t n_rows);
int kge_inspect(const int64_t *const *parts, const int64_t *part_len, int n_parts,
                int64_t n_rows, const kge_inspection *out, void *workspace,
                size_t workspace_bytes, void *stream);

/*
 * Several inspections in one call (at most 4 jobs).  Index sets of up to 65536 ids share
 * their kernel launches (one per radix digit pass plus one for the dedup); larger sets run
 * the multi-block sort one after the other.  Same outputs as kge_inspect.  A training step inspects concat(h, t, neg)
 * and r together this way.
 */
typedef struct kge_inspect_job {
    const int64_t *parts[4];  /* device pointers of the concatenated index arrays */
    int64_t part_len[4];
    int32_t n_parts;
    int32_t reserved;
    int64_t n_rows;
    kge_inspection out;
    void *workspace;          /* kge_inspect_workspace(n, n_rows) bytes, 16-byte aligned */
    size_t workspace_bytes;
} kge_inspect_job;
int kge_inspect_batch(const kge_inspect_job *jobs, int n_jobs, void *stream);
/* 1 if a batch with these two jobs (see kge_batch.fuse_inspection) can have its inspection fused
   into the score kernels, else 0. */
int kge_fused_inspection_ok(const kge_tables *tab, const kge_batch *bat, const kge_inspect_job *jobs);
/* 1 if kge_score_fwd fills kge_batch.back_rows for this batch (TransR, relation inspection given, no shared
   negatives, row width a multiple of four and within the grouped kernels' range), else 0.  No counterpart in
   the reference. */
int kge_back_rows_ok(const kge_tables *tab, const kge_batch *bat);

/*
 * Margin-ranking loss over score pairs and its gradient:
 *   L = mean_{b,k} max(0, margin - sign * (pos[b] - neg[b][k]))
 * loss[1], dpos[B], dneg[B, N].  workspace: kge_margin_loss_workspace(B, N) bytes.
 */
size_t kge_margin_loss_workspace(int64_t batch, int64_t n_neg);
int kge_margin_loss(const float *pos, const float *neg, int64_t batch, int64_t n_neg,
                    float margin, float sign, float *loss, float *dpos, float *dneg,
                    void *workspace, size_t workspace_bytes, void *stream);

/*
 * kge_margin_loss for callers that cannot allocate device memory (code under HIP graph capture,
 * tight serving loops, harnesses that forbid hipMalloc): same arguments and results, but the
 * per-row partial losses live in a device array built into the library (8 bytes per row,
 * KGE_MARGIN_LOSS_STATIC_MAX_BATCH rows = 512 KiB held on every GPU the library runs on until the
 * process ends) instead of a caller-provided workspace.  Allocates nothing.  batch above the
 * limit returns KGE_EWORKSPACE.  All calls on one GPU share that array: calls that overlap on one
 * GPU (different streams or threads) race; calls on one stream do not.  No counterpart in the
 * reference.
 */
#define KGE_MARGIN_LOSS_STATIC_MAX_BATCH 65536
int kge_margin_loss_static(const float *pos, const float *neg, int64_t batch, int64_t n_neg,
                           float margin, float sign, float *loss, float *dpos, float *dneg,
                           void *stream);

/*
 * Backward of kge_score_fwd: upstream dpos[B] (may be NULL = 0), dneg[B, n_neg]
 * -> one gradient row per unique table row, written once, no atomics.
 * The reference only prints per-triple dense gradient kernels
 * (apps/kge/kge.py:393-515); this entry point is what a training step needs
 * in their place.
 */
size_t kge_score_bwd_workspace(const kge_tables *tab, const kge_batch *bat);
int kge_score_bwd(const kge_tables *tab, const kge_batch *bat, const kge_saved *saved,
                  const float *dpos, const float *dneg, const kge_grads *grads,
                  void *workspace, size_t workspace_bytes, void *stream);

/*
 * Chunk-of-16 relation cache index, same outputs as the reference's
 * gpu_sort(relation, r_Uniq, r_Buffer, uniq_cnt, batch, rel_num)
 * (apps/kge/inspection/inspector.cu:68-143): r[batch] sorted ascending,
 * uniq[batch/16][16], buf[batch/16][16], cnt[batch/16] caller-zeroed int64.
 */
int kge_build_index(const int64_t *r, int64_t *uniq, int64_t *buf, int64_t *cnt, int64_t batch,
                    int64_t rel_num, void *stream);

/*
 * Shared negatives written out as explicit triples, the way the reference's neg_transR defines
 * them (apps/examples/examples.py:1447-1480: every view is flattened to batch * blocksize rows).
 * Outputs have B * (1 + n_neg) entries: the B positives first, then row B + b * n_neg + k =
 * (h[b], r[b], neg[(b / chunk) * n_neg + k]).  TransR and RESCAL have grouped forms of kge_score_fwd
 * (see there) and use the list only for what those do not take: shapes outside the grouped kernels.
 */
int kge_flatten_negatives(const kge_batch *bat, int64_t *h_flat, int64_t *r_flat, int64_t *t_flat,
                          void *stream);

/*
 * Sparse optimizer step on one table from (unique ids, gradient rows) as kge_score_bwd leaves
 * them: the step after backward.  The reference has no optimizer; these are the two row-wise
 * rules of the DGL-KE lineage its data layer comes from.  ids are distinct, so rows never collide.
 *   SGD      table[id] -= lr * g
 *   Adagrad  state[id] += mean(g^2);  table[id] -= lr * g / (sqrt(state[id]) + eps)
 * num_unique is the device scalar of the inspection; capacity = rows allocated behind ids/rows.
 */
int kge_sparse_sgd(float *table, int64_t dim, const int64_t *ids, const int32_t *num_unique, int64_t capacity,
                   const float *rows, float lr, void *stream);
int kge_sparse_adagrad(float *table, float *state, int64_t dim, const int64_t *ids, const int32_t *num_unique,
                       int64_t capacity, const float *rows, float lr, float eps, void *stream);

/*
 * The same two rules on the projection table of TransR / RESCAL (proj: [n_rel, dim, dim]) from gradients
 * that kge_score_bwd left partly factored (kge_grads.aux_x / aux_q / aux_factor_max, groups delimited by
 * rel_insp): a factored group's update is applied as  Proj[id] -= scale * sum_p x_p^T q_p  straight from
 * its rows, a dense group's from grads->aux_rows[u].  Adagrad's row statistic mean(g^2) of a factored
 * group is sum_{p,p'} (x_p . x_p')(q_p . q_p') / dim^2, the squared Frobenius norm of the sum of outer
 * products.  state: [n_rel].  With aux_factor_max = 0 both reduce to kge_sparse_sgd / kge_sparse_adagrad
 * on aux_rows.  dim % 4 == 0, 16-byte aligned arrays.
 */
int kge_sparse_sgd_factored(float *proj, int64_t dim, const kge_inspection *rel_insp, const kge_grads *grads,
                            float lr, void *stream);
int kge_sparse_adagrad_factored(float *proj, float *state, int64_t dim, const kge_inspection *rel_insp,
                                const kge_grads *grads, float lr, float eps, void *stream);

/*
 * Uniform negative entity ids for one batch, drawn on the device: out[i] for i < count is
 *   mulhi64(splitmix64(seed ^ splitmix64(step) ^ (i * 0x9E3779B97F4A7C15)), n_ent)
 * with splitmix64 the usual 64-bit finaliser.  Deterministic in (seed, step, i), no state, no
 * exclusion of true positives (the reference's sampler is created with exclude_positive=False,
 * apps/kge/data/data_init.py:26-43).  Stands where the reference calls the DGL EdgeSampler
 * (apps/kge/data/sampler.py:342-353) for the chunked negative tails.
 */
int kge_sample_negatives(int64_t *out, int64_t count, int64_t n_ent, uint64_t seed, uint64_t step, void *stream);

/*
 * One step of a staged training loop in ONE call (host-side sequencing only; no counterpart in the
 * reference, which has no training loop).  It enqueues what a host loop would enqueue with seven to ten
 * calls: on `side_stream` the inspection of the NEXT batch (TransR / RESCAL without negatives: both
 * inspections in one batch of launches, then the tile plans into next->fwd_workspace), on `stream` the step
 * of the CURRENT batch -- kge_score_fwd, kge_margin_loss when buf->loss is set, kge_score_bwd -- and the
 * events between the two streams.  For steps so short (tens of microseconds) that the host's per-call
 * overhead, not the device, would set the pace.
 *   cur == NULL   only stage `next` (in front of the first step);  next == NULL   only run `cur`.
 * A kge_step_batch keeps what belongs to one batch across steps: its index arrays and inspections
 * (bat.insp_jobs[0] = the entity index set, [1] = the relations; bat.ent_insp / rel_insp point to their
 * `out`), and three events the caller creates once (hipEventCreate; default flags are fine):
 *   inspected  recorded on side_stream behind the batch's inspection; kge_score_bwd waits for it right
 *              before its segmented reduction (kge_batch.insp_ready).  TransR / RESCAL without negatives:
 *              `stream` waits for it once, before the forward pass (it is recorded behind the plans too, and
 *              the batch was staged a step ahead), and kge_score_bwd has no wait of its own.
 *   planned    TransR / RESCAL without negatives: recorded behind the inspections and the tile plans.  Else
 *              unused (may be NULL).
 *   released   recorded on `stream` behind the step; a later staging of the same kge_step_batch makes
 *              side_stream wait for it before it overwrites the inspection (released_valid says whether
 *              it has been recorded yet; zero-initialise it).
 * Scores, gradients and workspaces (kge_step_buffers) are shared by all batches; sizes as for the
 * individual calls.  buf->loss == NULL: dpos / dneg are the caller's upstream gradients (inputs).
 * Results are those of the individual calls, bit for bit (the same launches in the same order).
 */
typedef struct kge_step_batch {
    kge_batch bat;
    void *fwd_workspace;        /* TransR / RESCAL without negatives: this batch's own forward workspace (plans), else NULL */
    size_t fwd_workspace_bytes;
    void *inspected, *planned, *released;  /* hipEvent_t */
    int32_t released_valid;
    int32_t reserved;
} kge_step_batch;

typedef struct kge_step_buffers {
    float *pos, *neg, *side_pos, *side_neg, *residual;  /* as kge_score_fwd */
    void *fwd_workspace;        /* for batches without one of their own */
    size_t fwd_workspace_bytes;
    float *loss;                /* [1] or NULL */
    float margin, sign;
    void *loss_workspace;
    size_t loss_workspace_bytes;
    float *dpos, *dneg;         /* [B], [B, n_neg] (either may be NULL = 0 where kge_score_bwd allows it) */
    kge_grads grads;
    void *bwd_workspace;
    size_t bwd_workspace_bytes;
} kge_step_buffers;

int kge_train_step_staged(const kge_tables *tab, kge_step_batch *cur, kge_step_batch *next, const kge_step_buffers *buf,
                          void *stream, void *side_stream);

/* Sets flag[0] (int32, caller-zeroed) to 1 if any idx[i] is outside [0, n_rows). */
int kge_check_indices(const int64_t *idx, int64_t n, int64_t n_rows, int32_t *flag, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* KGE_MI355_H */
