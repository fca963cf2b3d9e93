/*
 * CPU oracle for the KGE score-function path.  TEST INFRASTRUCTURE ONLY.
 *
 * This file is the checker the HIP kernels are compared against.  It is never
 * part of the shipped path: only tests, the smoke check and the benchmark's
 * cpu_baseline leg may load it.
 *
 * What it restates (all paths relative to the reference checkout):
 *   - the serial loop nests cuke's codegen.cpu emits for the KGE score
 *     functions: fp32 accumulators that start at 0 and are updated with
 *     `+=` in ascending index order, multiply then add (no FMA contraction)
 *       pycuke1/asg2ir.py:222-308   elementwise arithmetic -> loop nest
 *       pycuke1/asg2ir.py:407-525   einsum -> loops, `init = 0`, `+=`
 *       pycuke1/asg2ir.py:561-600   index -> inlined gather E[h[b]][j]
 *       pycuke1/codegen/cpu.py:23-107, apps/kge/README.md:37-79 (TransE text)
 *   - the model definitions
 *       apps/kge/kge.py:273-293  transE   (E[h]-E[t])+R[r]
 *       apps/kge/kge.py:296-318  transH   vh-vt+vr - bsv(bvv(vp,vh-vt),vp)
 *       apps/kge/kge.py:321-343  transR   bvm(vh-vt, Proj[r]) + vr
 *       apps/kge/kge.py:346-366  transF   bvv(vh+vr,vt)+bvv(vt-vr,vh)
 *       apps/kge/kge.py:369-390  RESCAL   bvv(bvm(vh,Proj[r]),vt)
 *       apps/kge/test_pytorch.py:21,40,58,74,91  (the same as eager formulas)
 *   - shared negatives: apps/examples/examples.py:1404-1444 (neg_transE):
 *       out[b][k] = f(E[h[b]], R[r[b]], E[tail[(b/C)*N + k]])
 *
 * Not in the reference (stated here, pinned by the CPU tests against torch
 * fp64 library routines, closed forms and finite differences): Lp norms of
 * the residual, DistMult, ComplEx, RotatE, the margin-ranking loss and every
 * gradient.  Gradients are derived from the forward definitions above, not
 * from apps/kge/kge.py:393-515 (those are print-only and partly transposed).
 *
 * Build: see oracle/Makefile (gcc -O2 -ffp-contract=off; no -ffast-math).
 */
#include <math.h>
#include <stddef.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

enum {
    ORC_TRANSE = 0,
    ORC_TRANSH = 1,
    ORC_TRANSR = 2,
    ORC_DISTMULT = 3,
    ORC_COMPLEX = 4,
    ORC_ROTATE = 5,
    ORC_TRANSF = 6,
    ORC_RESCAL = 7
};

/* floats per relation row / per aux row for a model of entity width d */
static int64_t rel_width(int model, int64_t d)
{
    switch (model) {
    case ORC_ROTATE: return d / 2;
    case ORC_RESCAL: return 0;
    default: return d;
    }
}
static int64_t aux_width(int model, int64_t d)
{
    switch (model) {
    case ORC_TRANSH: return d;
    case ORC_TRANSR:
    case ORC_RESCAL: return d * d;
    default: return 0;
    }
}

/* ---- residual vectors: what the reference's generated code returns -------- */

/* kge.py:289-290 / README.md:65-79: arr[b][j] = (E[h][j] - E[t][j]) + R[r][j] */
static void residual_transe(int64_t d, const float *eh, const float *rr, const float *et, float *out)
{
    for (int64_t j = 0; j < d; ++j) out[j] = (eh[j] - et[j]) + rr[j];
}

/* kge.py:315: vh - vt + vr - bsv(bvv(vp, vh - vt), vp).
 * bvv = einsum('i,i->') -> scalar starts at 0, += P[i]*d[i] ascending. */
static float residual_transh(int64_t d, const float *eh, const float *rr, const float *et,
                             const float *w, float *out)
{
    float s = 0.0f;
    for (int64_t i = 0; i < d; ++i) {
        float di = eh[i] - et[i];
        s += w[i] * di;
    }
    for (int64_t j = 0; j < d; ++j) out[j] = ((eh[j] - et[j]) + rr[j]) - s * w[j];
    return s;
}

/* kge.py:340: bvm(vh - vt, mr) + vr, einsum('i,ij->j'): j outer, i inner
 * (asg2ir.py:423-461: output indices first, then reduction indices). */
static void residual_transr(int64_t d, const float *eh, const float *rr, const float *et,
                            const float *m, float *out)
{
    for (int64_t j = 0; j < d; ++j) {
        float acc = 0.0f;
        for (int64_t i = 0; i < d; ++i) acc += (eh[i] - et[i]) * m[i * d + j];
        out[j] = acc + rr[j];
    }
}

int orc_residual(int model, int64_t B, int64_t d, const float *E, const float *R, const float *A,
                 const int64_t *h, const int64_t *r, const int64_t *t, float *out)
{
    for (int64_t b = 0; b < B; ++b) {
        const float *eh = E + h[b] * d, *et = E + t[b] * d, *rr = R + r[b] * d;
        float *o = out + b * d;
        switch (model) {
        case ORC_TRANSE: residual_transe(d, eh, rr, et, o); break;
        case ORC_TRANSH: residual_transh(d, eh, rr, et, A + r[b] * d, o); break;
        case ORC_TRANSR: residual_transr(d, eh, rr, et, A + r[b] * d * d, o); break;
        default: return -1;
        }
    }
    return 0;
}

/* ---- scalar scores -------------------------------------------------------- */

static float lp_norm(int p, int64_t d, const float *u)
{
    float s = 0.0f;
    if (p == 1) {
        for (int64_t j = 0; j < d; ++j) s += fabsf(u[j]);
        return s;
    }
    for (int64_t j = 0; j < d; ++j) s += u[j] * u[j];
    return sqrtf(s);
}

/* One triple.  tmp: d floats of scratch. */
static float score_one(int model, int p, float gamma, int64_t d, const float *eh, const float *rr,
                       const float *et, const float *aux, float *tmp)
{
    const int64_t half = d / 2;
    float s = 0.0f;
    switch (model) {
    case ORC_TRANSE:
        residual_transe(d, eh, rr, et, tmp);
        return lp_norm(p, d, tmp);
    case ORC_TRANSH:
        residual_transh(d, eh, rr, et, aux, tmp);
        return lp_norm(p, d, tmp);
    case ORC_TRANSR:
        residual_transr(d, eh, rr, et, aux, tmp);
        return lp_norm(p, d, tmp);
    case ORC_DISTMULT:
        for (int64_t i = 0; i < d; ++i) s += (eh[i] * rr[i]) * et[i];
        return s;
    case ORC_COMPLEX:
        /* rows are [re | im]; s = Re(<h, r, conj(t)>) */
        for (int64_t i = 0; i < half; ++i) {
            float hr = eh[i], hi = eh[half + i], qr = rr[i], qi = rr[half + i];
            float tr = et[i], ti = et[half + i];
            s += ((hr * qr) * tr + (hr * qi) * ti + (hi * qr) * ti) - (hi * qi) * tr;
        }
        return s;
    case ORC_ROTATE:
        /* entity rows [re | im], relation row = phase; s = gamma - sum |h e^{i th} - t| */
        for (int64_t i = 0; i < half; ++i) {
            float c = cosf(rr[i]), sn = sinf(rr[i]);
            float ur = (eh[i] * c - eh[half + i] * sn) - et[i];
            float ui = (eh[i] * sn + eh[half + i] * c) - et[half + i];
            s += sqrtf(ur * ur + ui * ui);
        }
        return gamma - s;
    case ORC_TRANSF: {
        /* kge.py:363: bvv(vh+vr, vt) + bvv(vt-vr, vh) */
        float s1 = 0.0f, s2 = 0.0f;
        for (int64_t i = 0; i < d; ++i) s1 += (eh[i] + rr[i]) * et[i];
        for (int64_t i = 0; i < d; ++i) s2 += (et[i] - rr[i]) * eh[i];
        return s1 + s2;
    }
    case ORC_RESCAL:
        /* kge.py:387: bvv(bvm(vh, mr), vt) */
        for (int64_t j = 0; j < d; ++j) {
            float acc = 0.0f;
            for (int64_t i = 0; i < d; ++i) acc += eh[i] * aux[i * d + j];
            tmp[j] = acc;
        }
        for (int64_t j = 0; j < d; ++j) s += tmp[j] * et[j];
        return s;
    default:
        return NAN;
    }
}

/* pos[B]; negs[B*N] when neg != NULL: positive b of chunk c = b / C is scored
 * against the N entities neg[c*N .. c*N+N-1] (examples.py:1404-1444 layout), which replace the
 * tail (neg_head == 0: triple (h_b, r_b, neg_k), the reference's layout) or the head
 * (neg_head != 0: triple (neg_k, r_b, t_b), the head batches of apps/kge/data/sampler.py). */
int orc_score(int model, int p, float gamma, int64_t B, int64_t d, const float *E, const float *R,
              const float *A, const int64_t *h, const int64_t *r, const int64_t *t,
              const int64_t *neg, int64_t C, int64_t N, int neg_head, float *pos, float *negs)
{
    const int64_t rw = rel_width(model, d), aw = aux_width(model, d);
    float *tmp = (float *)malloc(sizeof(float) * (size_t)(d > 0 ? d : 1));
    if (!tmp) return -2;
#ifdef _OPENMP
#pragma omp parallel
    {
        float *ltmp = (float *)malloc(sizeof(float) * (size_t)(d > 0 ? d : 1));
#pragma omp for schedule(static)
        for (int64_t b = 0; b < B; ++b) {
            const float *eh = E + h[b] * d, *rr = R ? R + r[b] * rw : NULL;
            const float *ax = A ? A + r[b] * aw : NULL;
            if (pos) pos[b] = score_one(model, p, gamma, d, eh, rr, E + t[b] * d, ax, ltmp);
            if (neg) {
                const int64_t c = b / C;
                for (int64_t k = 0; k < N; ++k) {
                    const float *en = E + neg[c * N + k] * d;
                    negs[b * N + k] = neg_head ? score_one(model, p, gamma, d, en, rr, E + t[b] * d, ax, ltmp)
                                               : score_one(model, p, gamma, d, eh, rr, en, ax, ltmp);
                }
            }
        }
        free(ltmp);
    }
#else
    for (int64_t b = 0; b < B; ++b) {
        const float *eh = E + h[b] * d, *rr = R ? R + r[b] * rw : NULL;
        const float *ax = A ? A + r[b] * aw : NULL;
        if (pos) pos[b] = score_one(model, p, gamma, d, eh, rr, E + t[b] * d, ax, tmp);
        if (neg) {
            const int64_t c = b / C;
            for (int64_t k = 0; k < N; ++k) {
                const float *en = E + neg[c * N + k] * d;
                negs[b * N + k] = neg_head ? score_one(model, p, gamma, d, en, rr, E + t[b] * d, ax, tmp)
                                           : score_one(model, p, gamma, d, eh, rr, en, ax, tmp);
            }
        }
    }
#endif
    free(tmp);
    return 0;
}

/* ---- gradients ------------------------------------------------------------ */

/* q = g * d||u||_p/du ; sign(0) = 0 and a zero L2 norm gives a zero gradient */
static void lp_grad(int p, int64_t d, const float *u, float g, float *q)
{
    if (p == 1) {
        for (int64_t j = 0; j < d; ++j) q[j] = u[j] > 0.0f ? g : (u[j] < 0.0f ? -g : 0.0f);
        return;
    }
    float s = lp_norm(2, d, u);
    for (int64_t j = 0; j < d; ++j) q[j] = s > 0.0f ? g * (u[j] / s) : 0.0f;
}

/* One triple with upstream gradient g = dL/dscore; adds into dh, dr, dt, daux.
 * tmp: 3*d floats. */
static void bwd_one(int model, int p, int64_t d, const float *eh, const float *rr, const float *et,
                    const float *aux, float g, float *dh, float *dr, float *dt, float *daux,
                    float *tmp)
{
    const int64_t half = d / 2;
    float *u = tmp, *q = tmp + d, *x = tmp + 2 * d;
    switch (model) {
    case ORC_TRANSE:
        residual_transe(d, eh, rr, et, u);
        lp_grad(p, d, u, g, q);
        for (int64_t j = 0; j < d; ++j) {
            dh[j] += q[j];
            dr[j] += q[j];
            dt[j] -= q[j];
        }
        break;
    case ORC_TRANSH: {
        /* u = d0 + r - (w.d0) w ;  dL/dd0 = q - (q.w) w ;  dL/dw = -((q.w) d0 + (w.d0) q) */
        float sd = residual_transh(d, eh, rr, et, aux, u);
        lp_grad(p, d, u, g, q);
        /* q.w enters every element of the row: a rounding error in it is coherent across the
         * row and across the triples sharing w, so this scalar is reduced in double */
        double qwd = 0.0;
        for (int64_t j = 0; j < d; ++j) qwd += (double)q[j] * (double)aux[j];
        const float qw = (float)qwd;
        for (int64_t i = 0; i < d; ++i) {
            float gi = q[i] - qw * aux[i];
            dh[i] += gi;
            dt[i] -= gi;
            dr[i] += q[i];
            daux[i] -= qw * (eh[i] - et[i]) + sd * q[i];
        }
        break;
    }
    case ORC_TRANSR:
        /* e_j = sum_i d0_i M_ij + r_j ;  dd0_i = sum_j M_ij q_j ;  dM_ij = d0_i q_j */
        residual_transr(d, eh, rr, et, aux, u);
        lp_grad(p, d, u, g, q);
        for (int64_t i = 0; i < d; ++i) {
            double acc = 0.0;
            for (int64_t j = 0; j < d; ++j) acc += (double)aux[i * d + j] * (double)q[j];
            x[i] = (float)acc;
        }
        for (int64_t i = 0; i < d; ++i) {
            float d0 = eh[i] - et[i];
            dh[i] += x[i];
            dt[i] -= x[i];
            dr[i] += q[i];
            for (int64_t j = 0; j < d; ++j) daux[i * d + j] += d0 * q[j];
        }
        break;
    case ORC_DISTMULT:
        for (int64_t i = 0; i < d; ++i) {
            dh[i] += g * (rr[i] * et[i]);
            dr[i] += g * (eh[i] * et[i]);
            dt[i] += g * (eh[i] * rr[i]);
        }
        break;
    case ORC_COMPLEX:
        for (int64_t i = 0; i < half; ++i) {
            float hr = eh[i], hi = eh[half + i], qr = rr[i], qi = rr[half + i];
            float tr = et[i], ti = et[half + i];
            dh[i] += g * (qr * tr + qi * ti);
            dh[half + i] += g * (qr * ti - qi * tr);
            dr[i] += g * (hr * tr + hi * ti);
            dr[half + i] += g * (hr * ti - hi * tr);
            dt[i] += g * (hr * qr - hi * qi);
            dt[half + i] += g * (hr * qi + hi * qr);
        }
        break;
    case ORC_ROTATE:
        /* s = gamma - sum m_i, m = |a - t|, a = h e^{i th};  ds/du = -u/m */
        for (int64_t i = 0; i < half; ++i) {
            float c = cosf(rr[i]), sn = sinf(rr[i]);
            float ar = eh[i] * c - eh[half + i] * sn, ai = eh[i] * sn + eh[half + i] * c;
            float ur = ar - et[i], ui = ai - et[half + i];
            float m = sqrtf(ur * ur + ui * ui);
            float qr = m > 0.0f ? -g * (ur / m) : 0.0f;
            float qi = m > 0.0f ? -g * (ui / m) : 0.0f;
            dh[i] += qr * c + qi * sn;
            dh[half + i] += qi * c - qr * sn;
            dt[i] -= qr;
            dt[half + i] -= qi;
            dr[i] += qi * ar - qr * ai;
        }
        break;
    case ORC_TRANSF:
        /* s = 2 h.t + r.t - r.h */
        for (int64_t i = 0; i < d; ++i) {
            dh[i] += g * (2.0f * et[i] - rr[i]);
            dt[i] += g * (2.0f * eh[i] + rr[i]);
            dr[i] += g * (et[i] - eh[i]);
        }
        break;
    case ORC_RESCAL:
        for (int64_t i = 0; i < d; ++i) {
            float acc = 0.0f;
            for (int64_t j = 0; j < d; ++j) acc += aux[i * d + j] * et[j];
            dh[i] += g * acc;
        }
        for (int64_t j = 0; j < d; ++j) {
            float acc = 0.0f;
            for (int64_t i = 0; i < d; ++i) acc += eh[i] * aux[i * d + j];
            dt[j] += g * acc;
        }
        for (int64_t i = 0; i < d; ++i)
            for (int64_t j = 0; j < d; ++j) daux[i * d + j] += g * (eh[i] * et[j]);
        break;
    default:
        break;
    }
}

/*
 * Sparse row gradients.  Every occurrence of a row is mapped by the caller to
 * an output row ("slot", e.g. numpy.unique's inverse): slot_h[B], slot_t[B],
 * slot_neg[n_chunks*N] index gE[U_e, d]; slot_r[B] indexes gR[U_r, rel_width]
 * and gA[U_r, aux_width].
 *
 * Each triple's contribution is computed in fp32 as bwd_one states it (its inner
 * contractions in double, rounded once);
 * the sum ACROSS triples (up to ~10^6 terms for a hot row) is accumulated in
 * double and rounded to fp32 once, so that the oracle stays a trustworthy
 * reference for long sums (a serial fp32 sum of n terms drifts by ~sqrt(n)
 * ulps of its partial sums, more than the parity bar for n > 10^4).
 * Order: b ascending; for each b the positive first, then k ascending.
 */
static void add_row(double *acc, const float *src, int64_t n)
{
    for (int64_t i = 0; i < n; ++i) acc[i] += (double)src[i];
}

/* The triples order[i] (or i itself without an order) for b0 <= i < b1, accumulated into aE / aR / aA
 * (double).  tmp: 3d + 1 floats, one: 3d + aux_width + 1 floats. */
static void bwd_range(int model, int p, const int64_t *order, int64_t b0, int64_t b1, int64_t d, const float *E, const float *R,
                      const float *A, const int64_t *h, const int64_t *r, const int64_t *t,
                      const int64_t *neg, int64_t C, int64_t N, int neg_head, const float *dpos, const float *dneg,
                      const int64_t *slot_h, const int64_t *slot_t, const int64_t *slot_neg,
                      const int64_t *slot_r, double *aE, double *aR, double *aA, float *tmp, float *one)
{
    const int64_t rw = rel_width(model, d), aw = aux_width(model, d);
    float *dh = one, *dr = one + d, *dt = one + 2 * d, *da = one + 3 * d;
    for (int64_t i = b0; i < b1; ++i) {
        const int64_t b = order ? order[i] : i;
        const float *eh = E + h[b] * d, *rr = R ? R + r[b] * rw : NULL;
        const float *ax = A ? A + r[b] * aw : NULL;
        const int64_t n_t = 1 + ((neg && dneg) ? N : 0);
        const int64_t c = C > 0 ? b / C : 0;
        for (int64_t q = 0; q < n_t; ++q) {
            float g;
            const float *ehead = eh, *et = E + t[b] * d;
            int64_t slot_head = slot_h[b], slot_tail = slot_t[b];
            if (q == 0) {
                if (!dpos) continue;
                g = dpos[b];
            } else {  /* the negative replaces the tail, or the head when neg_head is set */
                const int64_t k = q - 1;
                g = dneg[b * N + k];
                if (neg_head) ehead = E + neg[c * N + k] * d, slot_head = slot_neg[c * N + k];
                else et = E + neg[c * N + k] * d, slot_tail = slot_neg[c * N + k];
            }
            memset(one, 0, sizeof(float) * (size_t)(3 * d + aw));
            bwd_one(model, p, d, ehead, rr, et, ax, g, dh, dr, dt, da, tmp);
            add_row(aE + slot_head * d, dh, d);
            add_row(aE + slot_tail * d, dt, d);
            if (rw) add_row(aR + slot_r[b] * rw, dr, rw);
            if (aw) add_row(aA + slot_r[b] * aw, da, aw);
        }
    }
}

/* With OpenMP (the timed multi-thread leg of the benchmark only; the checker is built without
 * it) the batch is cut into one contiguous range per thread, every thread accumulates into
 * double arrays of its own, and the per-thread arrays are added up in thread order.
 * The projection models (a d x d gradient per relation) are cut by RELATION instead: the triples are
 * ordered by relation slot, every thread takes a contiguous range of whole relations (balanced by
 * triple count) and accumulates their relation and projection rows straight into the one shared
 * array (no other thread touches those rows); only the entity rows are kept per thread.  A dense
 * n_slots_r x d x d double array per thread made that leg slower than one thread. */
int orc_backward(int model, int p, int64_t B, int64_t d, const float *E, const float *R,
                 const float *A, const int64_t *h, const int64_t *r, const int64_t *t,
                 const int64_t *neg, int64_t C, int64_t N, int neg_head, const float *dpos, const float *dneg,
                 const int64_t *slot_h, const int64_t *slot_t, const int64_t *slot_neg,
                 const int64_t *slot_r, int64_t n_slots_e, int64_t n_slots_r, float *gE, float *gR,
                 float *gA)
{
    const int64_t rw = rel_width(model, d), aw = aux_width(model, d);
    const size_t nE = (size_t)(n_slots_e * d + 1), nR = (size_t)(n_slots_r * rw + 1), nA = (size_t)(n_slots_r * aw + 1);
    int T = 1;
#ifdef _OPENMP
    extern int omp_get_max_threads(void);
    extern int omp_get_thread_num(void);
    T = omp_get_max_threads();
    if (T > B) T = B > 0 ? (int)B : 1;
#endif
    const int by_relation = T > 1 && aw == d * d && n_slots_r > 0;
    const int TR = by_relation ? 1 : T;  /* copies of the relation-side accumulators */
    double *aE = (double *)calloc(nE * (size_t)T, sizeof(double));
    double *aR = (double *)calloc(nR * (size_t)TR, sizeof(double));
    double *aA = (double *)calloc(nA * (size_t)TR, sizeof(double));
    int64_t *order = NULL, *cut = NULL;
    if (by_relation) {  /* counting sort of the triples by relation slot; cut[q] = first position of thread q */
        order = (int64_t *)malloc(sizeof(int64_t) * (size_t)(B + 1));
        cut = (int64_t *)malloc(sizeof(int64_t) * (size_t)(T + 1));
        int64_t *start = (int64_t *)calloc((size_t)(n_slots_r + 1), sizeof(int64_t));
        if (order && cut && start) {
            for (int64_t b = 0; b < B; ++b) start[slot_r[b] + 1]++;
            for (int64_t u = 0; u < n_slots_r; ++u) start[u + 1] += start[u];
            int q = 0;
            cut[0] = 0;
            for (int64_t u = 0; u < n_slots_r && q + 1 < T; ++u)  /* thread q ends at the relation boundary nearest to its share */
                while (q + 1 < T && start[u + 1] >= B * (q + 1) / T) cut[++q] = start[u + 1];
            while (q < T) cut[++q] = B;
            int64_t *fill = (int64_t *)malloc(sizeof(int64_t) * (size_t)(n_slots_r + 1));
            if (fill) {
                memcpy(fill, start, sizeof(int64_t) * (size_t)(n_slots_r + 1));
                for (int64_t b = 0; b < B; ++b) order[fill[slot_r[b]]++] = b;
                free(fill);
            } else {
                free(order);
                order = NULL;
            }
        }
        free(start);
    }
    if (!aE || !aR || !aA || (by_relation && (!order || !cut))) {
        free(aE); free(aR); free(aA); free(order); free(cut);
        return -2;
    }
    int failed = 0;
#ifdef _OPENMP
#pragma omp parallel num_threads(T)
#endif
    {
        int tid = 0;
#ifdef _OPENMP
        tid = omp_get_thread_num();
#endif
        float *tmp = (float *)malloc(sizeof(float) * (size_t)(3 * d + 1));
        float *one = (float *)malloc(sizeof(float) * (size_t)(3 * d + aw + 1)); /* dh | dr | dt | daux */
        if (!tmp || !one) {
            failed = 1;
        } else {
            const int64_t b0 = by_relation ? cut[tid] : B * tid / T, b1 = by_relation ? cut[tid + 1] : B * (tid + 1) / T;
            const size_t rel_copy = by_relation ? 0 : (size_t)tid;
            bwd_range(model, p, order, b0, b1, d, E, R, A, h, r, t, neg, C, N, neg_head, dpos, dneg, slot_h, slot_t,
                      slot_neg, slot_r, aE + nE * (size_t)tid, aR + nR * rel_copy, aA + nA * rel_copy, tmp, one);
        }
        free(tmp);
        free(one);
    }
    free(order);
    free(cut);
    if (failed) {
        free(aE); free(aR); free(aA);
        return -2;
    }
#ifdef _OPENMP
#pragma omp parallel for schedule(static)
#endif
    for (int64_t i = 0; i < n_slots_e * d; ++i) {
        double s = aE[i];
        for (int q = 1; q < T; ++q) s += aE[nE * (size_t)q + (size_t)i];
        gE[i] = (float)s;
    }
    if (gR) {
        for (int64_t i = 0; i < n_slots_r * rw; ++i) {
            double s = aR[i];
            for (int q = 1; q < TR; ++q) s += aR[nR * (size_t)q + (size_t)i];
            gR[i] = (float)s;
        }
    }
    if (gA) {
#ifdef _OPENMP
#pragma omp parallel for schedule(static)
#endif
        for (int64_t i = 0; i < n_slots_r * aw; ++i) {
            double s = aA[i];
            for (int q = 1; q < TR; ++q) s += aA[nA * (size_t)q + (size_t)i];
            gA[i] = (float)s;
        }
    }
    free(aE); free(aR); free(aA);
    return 0;
}

/*
 * Which gradient rows an L1 sign ambiguity can reach.  The L1 gradient of TransE / TransH is a
 * sum of signs of residual elements; an element within rounding of zero may get either sign
 * from two correct fp32 implementations, and (TransH) one flipped sign moves every column of
 * the rows of that triple through q.w.  For every triple and pair of the batch whose residual
 * holds an element with |u_j| <= eps this marks the slots of its head, tail / negative and
 * relation rows by adding the number of such elements to cntE[n_slots_e] / cntR[n_slots_r]
 * (int32, caller-zeroed): a row's count bounds how many sign flips can reach that row.  Returns
 * the total number of such elements, -1 for a model without an L1 form.
 */
int64_t orc_l1_ambiguous(int model, int64_t B, int64_t d, const float *E, const float *R, const float *A,
                         const int64_t *h, const int64_t *r, const int64_t *t, const int64_t *neg, int64_t C,
                         int64_t N, int neg_head, float eps, const int64_t *slot_h, const int64_t *slot_t,
                         const int64_t *slot_neg, const int64_t *slot_r, int32_t *cntE, int32_t *cntR)
{
    if (model != ORC_TRANSE && model != ORC_TRANSH) return -1;
    int64_t total = 0;
#ifdef _OPENMP
#pragma omp parallel reduction(+ : total)
#endif
    {
        float *u = (float *)malloc(sizeof(float) * (size_t)(d + 1));
#ifdef _OPENMP
#pragma omp for schedule(static)
#endif
        for (int64_t b = 0; b < B; ++b) {
            const float *rr = R + r[b] * d, *ax = A ? A + r[b] * d : NULL;
            const int64_t c = C > 0 ? b / C : 0;
            for (int64_t q = 0; q < 1 + (neg ? N : 0); ++q) {
                const float *eh = E + h[b] * d, *et = E + t[b] * d;
                int64_t sh = slot_h[b], st = slot_t[b];
                if (q > 0) {
                    const int64_t k = q - 1;
                    if (neg_head) eh = E + neg[c * N + k] * d, sh = slot_neg[c * N + k];
                    else et = E + neg[c * N + k] * d, st = slot_neg[c * N + k];
                }
                if (model == ORC_TRANSE) residual_transe(d, eh, rr, et, u);
                else (void)residual_transh(d, eh, rr, et, ax, u);
                int64_t n = 0;
                for (int64_t j = 0; j < d; ++j) n += fabsf(u[j]) <= eps;
                if (n) {
#ifdef _OPENMP
#pragma omp atomic
#endif
                    cntE[sh] += (int32_t)n;
#ifdef _OPENMP
#pragma omp atomic
#endif
                    cntE[st] += (int32_t)n;
#ifdef _OPENMP
#pragma omp atomic
#endif
                    cntR[slot_r[b]] += (int32_t)n;
                    total += n;
                }
            }
        }
        free(u);
    }
    return total;
}

/*
 * Margin-ranking loss over positive/negative score pairs,
 *   L = mean_{b,k} max(0, margin - sign * (pos[b] - neg[b,k])),
 * sign = +1 when larger scores are better (== torch margin_ranking_loss with
 * y = 1), sign = -1 for distance scores.  The mean is accumulated in double.
 * Writes dL/dpos[B], dL/dneg[B*N].
 */
int orc_margin_loss(const float *pos, const float *neg, int64_t B, int64_t N, float margin,
                    float sign, float *loss, float *dpos, float *dneg)
{
    double acc = 0.0;
    const float inv = 1.0f / (float)(B * N);
    for (int64_t b = 0; b < B; ++b) {
        float cnt = 0.0f;
        for (int64_t k = 0; k < N; ++k) {
            float v = margin - sign * (pos[b] - neg[b * N + k]);
            int on = v > 0.0f;
            if (on) {
                acc += (double)v;
                cnt += 1.0f;
            }
            if (dneg) dneg[b * N + k] = on ? sign * inv : 0.0f;
        }
        if (dpos) dpos[b] = -sign * inv * cnt;
    }
    *loss = (float)(acc / (double)(B * N));
    return 0;
}

/*
 * Restatement of the reference's chunk-of-16 relation index builder
 * (apps/kge/inspection/inspector.cu:68-136) for well-formed chunks: r is
 * globally sorted (apps/kge/test_cuke.py:93-97), chunk = 16 consecutive ids.
 * The kernel's tournament (inspector.cu:102-114) is replayed literally so the
 * slot choice, including its heuristic second slot, matches.  A chunk with 16
 * distinct ids writes out of bounds in the reference (inspector.cu:90) and has
 * no defined result; this restatement reports it with return value 1 and
 * leaves that chunk's outputs as the untouched-zero / sentinel pattern the
 * in-bounds part of the kernel would give.
 */
int orc_build_index(const int64_t *r, int64_t batch, int64_t rel_num, int64_t *uniq, int64_t *buf,
                    int64_t *cnt)
{
    enum { CH = 16 };
    int any_undefined = 0;
    for (int64_t blk = 0; blk < batch / CH; ++blk) {
        int idx[CH], ord[CH], ibuf[CH], iuniq[CH + 1], pcount[CH + 1], ord_uniq[CH], count[CH],
            idx_count[CH];
        int pos[CH];
        for (int i = 0; i < CH; ++i) {
            idx[i] = (int)r[blk * CH + i];
            pos[i] = i;
            ord_uniq[i] = i;
            pcount[i] = 0;
            count[i] = -1;
            idx_count[i] = -1;
        }
        pcount[CH] = 0;
        /* bitonic_sort: ascending sort; ord[original position] = sorted position.
         * Any correct ascending sort gives the same sorted keys; equal keys are
         * indistinguishable afterwards because only their values are used. */
        for (int i = 1; i < CH; ++i) { /* insertion sort, stable */
            int kv = idx[i], pv = pos[i], j = i - 1;
            while (j >= 0 && idx[j] > kv) {
                idx[j + 1] = idx[j];
                pos[j + 1] = pos[j];
                --j;
            }
            idx[j + 1] = kv;
            pos[j + 1] = pv;
        }
        for (int i = 0; i < CH; ++i) ord[pos[i]] = i;
        /* run heads and their inclusive scan (inspector.cu:80-88) */
        ibuf[0] = 0;
        for (int i = 1; i < CH; ++i) ibuf[i] = ibuf[i - 1] + (idx[i] > idx[i - 1] ? 1 : 0);
        /* run boundaries (inspector.cu:90-93) */
        if (ibuf[CH - 1] + 1 >= CH) any_undefined = 1; /* pcount[16] write in the reference */
        pcount[ibuf[CH - 1] + 1] = CH;
        for (int i = 1; i < CH; ++i)
            if (idx[i] > idx[i - 1]) pcount[ibuf[i]] = i;
        for (int i = 0; i <= CH; ++i) iuniq[i] = (int)rel_num;
        /* run lengths (inspector.cu:97-100) */
        for (int i = 1; i < CH; ++i)
            if (pcount[i] - pcount[i - 1] > 0) {
                count[i - 1] = pcount[i] - pcount[i - 1];
                idx_count[i - 1] = pcount[i] - 1;
            }
        /* tournament (inspector.cu:102-109): lock-step halving compare-swap */
        for (int s = CH / 2; s > 0; s >>= 1)
            for (int i = 0; i < s; ++i)
                if (count[i] < count[i + s]) {
                    int tmpv;
                    tmpv = count[i], count[i] = count[i + s], count[i + s] = tmpv;
                    tmpv = idx_count[i], idx_count[i] = idx_count[i + s], idx_count[i + s] = tmpv;
                    tmpv = ord_uniq[i], ord_uniq[i] = ord_uniq[i + s], ord_uniq[i + s] = tmpv;
                }
        if (count[1] < count[2]) { /* inspector.cu:112-114 */
            int tmpv;
            tmpv = count[1], count[1] = count[2], count[2] = tmpv;
            tmpv = idx_count[1], idx_count[1] = idx_count[2], idx_count[2] = tmpv;
            tmpv = ord_uniq[1], ord_uniq[1] = ord_uniq[2], ord_uniq[2] = tmpv;
        }
        for (int i = 0; i < 2; ++i) /* inspector.cu:118-119, T = 2 */
            if (count[i] > 1) iuniq[i] = idx[idx_count[i]];
        int nb[CH];
        for (int i = 0; i < CH; ++i) { /* inspector.cu:122-130 */
            if (ibuf[i] == ord_uniq[0] && iuniq[0] < rel_num) nb[i] = 0;
            else if (ibuf[i] == ord_uniq[1] && iuniq[1] < rel_num) nb[i] = 1;
            else nb[i] = idx[i] + CH;
        }
        for (int i = 0; i < CH; ++i) /* inspector.cu:131-133 */
            if (iuniq[i] < rel_num && iuniq[i + 1] == rel_num) cnt[blk] = i + 1;
        for (int i = 0; i < CH; ++i) {
            buf[blk * CH + i] = nb[ord[i]];
            uniq[blk * CH + i] = iuniq[i];
        }
    }
    return any_undefined;
}

/*
 * Sparse optimizer steps (not in the reference; DGL-KE's row-wise rules, see the C header of the
 * library).  ids are distinct.  Pinned in the tests against numpy fancy-indexing formulas.
 */
int orc_sparse_sgd(float *table, int64_t d, const int64_t *ids, int64_t n, const float *rows, float lr)
{
    for (int64_t u = 0; u < n; ++u)
        for (int64_t j = 0; j < d; ++j) table[ids[u] * d + j] -= lr * rows[u * d + j];
    return 0;
}

int orc_sparse_adagrad(float *table, float *state, int64_t d, const int64_t *ids, int64_t n, const float *rows,
                       float lr, float eps)
{
    for (int64_t u = 0; u < n; ++u) {
        float sq = 0.0f;
        for (int64_t j = 0; j < d; ++j) sq += rows[u * d + j] * rows[u * d + j];
        state[ids[u]] += sq / (float)d;
        const float scale = lr / (sqrtf(state[ids[u]]) + eps);
        for (int64_t j = 0; j < d; ++j) table[ids[u] * d + j] -= scale * rows[u * d + j];
    }
    return 0;
}

int orc_threads(void)
{
#ifdef _OPENMP
    extern int omp_get_max_threads(void);
    return omp_get_max_threads();
#else
    return 1;
#endif
}
