// The per-positive score kernels' body (one wavefront per (h, r, t) triple), shared by the
// launch of its own (score_pos.hip) and by the shared-negative tile launches that carry the
// positives of DistMult / ComplEx along (score_neg.hip).
#pragma once

#include "common.hpp"

namespace kge {

struct PosArgs {
    const float *ent, *rel, *aux;
    const int64_t *h, *r, *t;
    int64_t B;
    int d, rel_dim;
    float gamma;
    float *pos;       // [B] scores or nullptr
    float *resid;     // [B, d] or nullptr: residual rows (TransE / TransH / TransR), the projected heads
                      // E[h] Proj[r] (RESCAL) or, for RotatE, the rotated heads h e^{i theta} laid out [re | im]
    float *side_pos;  // [B] TransH: w.h; TransF: r.h (used by the shared-negative kernels)
    int head;         // negatives replace the head: side_pos = w.t / r.t, RotatE resid = t e^{-i theta}
};

constexpr int kPosWaves = 4;

template <int P>
__device__ __forceinline__ float norm_term(float u)
{
    return P == 1 ? fabsf(u) : u * u;
}

// The work of one workgroup of kPosWaves positives: block `blk` takes the positives
// blk * kPosWaves .. + kPosWaves - 1.  `lds`: kPosWaves * d floats for TransR / RESCAL, else unused.
template <int MODEL, int P, int V>
__device__ __forceinline__ void score_pos_body(const PosArgs &a, float *lds, int64_t blk)
{
    const int lane = threadIdx.x & (kWave - 1);
    const int wave = threadIdx.x >> 6;
    const int64_t b = blk * kPosWaves + wave;
    const bool valid = b < a.B;
    const int64_t bb = valid ? b : 0;
    const int d = a.d;
    const int64_t rid = a.r[bb];
    const float *eh = a.ent + a.h[bb] * (int64_t)d;
    const float *et = a.ent + a.t[bb] * (int64_t)d;
    const float *rr = a.rel ? a.rel + rid * (int64_t)a.rel_dim : nullptr;
    float *out = a.resid ? a.resid + bb * (int64_t)d : nullptr;
    float acc = 0.0f;

    if constexpr (MODEL == KGE_TRANSE) {
        for (int j = lane * V; j < d; j += kWave * V) {
            const Vec<V> vh = Vec<V>::load(eh + j), vt = Vec<V>::load(et + j),
                         vr = Vec<V>::load(rr + j);
            Vec<V> u;
#pragma unroll
            for (int e = 0; e < V; ++e) {
                u.v[e] = (vh.v[e] - vt.v[e]) + vr.v[e];  // same order as the generated loop
                acc += norm_term<P>(u.v[e]);
            }
            if (out && valid) u.store(out + j);
        }
    } else if constexpr (MODEL == KGE_TRANSH) {
        const float *w = a.aux + rid * (int64_t)d;
        float sd = 0.0f, wh = 0.0f;
        for (int j = lane * V; j < d; j += kWave * V) {
            const Vec<V> vh = Vec<V>::load(eh + j), vt = Vec<V>::load(et + j),
                         vw = Vec<V>::load(w + j);
#pragma unroll
            for (int e = 0; e < V; ++e) {
                sd += vw.v[e] * (vh.v[e] - vt.v[e]);
                wh += vw.v[e] * (a.head ? vt.v[e] : vh.v[e]);
            }
        }
        sd = wave_sum(sd);
        wh = wave_sum(wh);
        if (a.side_pos && valid && lane == 0) a.side_pos[b] = wh;
        for (int j = lane * V; j < d; j += kWave * V) {
            const Vec<V> vh = Vec<V>::load(eh + j), vt = Vec<V>::load(et + j),
                         vr = Vec<V>::load(rr + j), vw = Vec<V>::load(w + j);
            Vec<V> u;
#pragma unroll
            for (int e = 0; e < V; ++e) {
                u.v[e] = ((vh.v[e] - vt.v[e]) + vr.v[e]) - sd * vw.v[e];
                acc += norm_term<P>(u.v[e]);
            }
            if (out && valid) u.store(out + j);
        }
    } else if constexpr (MODEL == KGE_TRANSR || MODEL == KGE_RESCAL) {
        // Ungrouped per-triple vector x matrix product (the shape of the reference's
        // kernel: every triple streams its own 4*d*d-byte projection).  The grouped MFMA
        // path in transr.hip is the fast one; this is the fallback without relation groups.
        const float *m = a.aux + rid * (int64_t)d * d;
        float *x = lds + wave * d;
        for (int i = lane; i < d; i += kWave) x[i] = MODEL == KGE_TRANSR ? eh[i] - et[i] : eh[i];
        __syncthreads();
        for (int j = lane * V; j < d; j += kWave * V) {
            Vec<V> s;
#pragma unroll
            for (int e = 0; e < V; ++e) s.v[e] = 0.0f;
            for (int i = 0; i < d; ++i) {
                const float xi = x[i];
                const Vec<V> vm = Vec<V>::load(m + (int64_t)i * d + j);
#pragma unroll
                for (int e = 0; e < V; ++e) s.v[e] += xi * vm.v[e];
            }
            if constexpr (MODEL == KGE_TRANSR) {
                const Vec<V> vr = Vec<V>::load(rr + j);
#pragma unroll
                for (int e = 0; e < V; ++e) {
                    s.v[e] += vr.v[e];
                    acc += norm_term<P>(s.v[e]);
                }
                if (out && valid) s.store(out + j);
            } else {
                const Vec<V> vt = Vec<V>::load(et + j);
#pragma unroll
                for (int e = 0; e < V; ++e) acc += s.v[e] * vt.v[e];
                if (out && valid) s.store(out + j);  // E[h] Proj[r], consumed by the backward pass
            }
        }
    } else if constexpr (MODEL == KGE_DISTMULT) {
        for (int j = lane * V; j < d; j += kWave * V) {
            const Vec<V> vh = Vec<V>::load(eh + j), vt = Vec<V>::load(et + j),
                         vr = Vec<V>::load(rr + j);
#pragma unroll
            for (int e = 0; e < V; ++e) acc += (vh.v[e] * vr.v[e]) * vt.v[e];
        }
    } else if constexpr (MODEL == KGE_TRANSF) {
        float rx = 0.0f;  // r . (the side the shared negatives keep)
        for (int j = lane * V; j < d; j += kWave * V) {
            const Vec<V> vh = Vec<V>::load(eh + j), vt = Vec<V>::load(et + j),
                         vr = Vec<V>::load(rr + j);
#pragma unroll
            for (int e = 0; e < V; ++e) {
                acc += (vh.v[e] + vr.v[e]) * vt.v[e] + (vt.v[e] - vr.v[e]) * vh.v[e];
                rx += vr.v[e] * (a.head ? vt.v[e] : vh.v[e]);
            }
        }
        if (a.side_pos) {  // uniform
            rx = wave_sum(rx);
            if (valid && lane == 0) a.side_pos[b] = rx;
        }
    } else if constexpr (MODEL == KGE_COMPLEX) {
        const int half = d / 2;
        for (int j = lane * V; j < half; j += kWave * V) {
            const Vec<V> hr = Vec<V>::load(eh + j), hi = Vec<V>::load(eh + half + j);
            const Vec<V> tr = Vec<V>::load(et + j), ti = Vec<V>::load(et + half + j);
            const Vec<V> qr = Vec<V>::load(rr + j), qi = Vec<V>::load(rr + half + j);
#pragma unroll
            for (int e = 0; e < V; ++e) {
                const float ar = hr.v[e] * qr.v[e] - hi.v[e] * qi.v[e];
                const float ai = hr.v[e] * qi.v[e] + hi.v[e] * qr.v[e];
                acc += ar * tr.v[e] + ai * ti.v[e];
            }
        }
    } else if constexpr (MODEL == KGE_ROTATE) {
        const int half = d / 2;
        for (int j = lane * V; j < half; j += kWave * V) {
            const Vec<V> hr = Vec<V>::load(eh + j), hi = Vec<V>::load(eh + half + j);
            const Vec<V> tr = Vec<V>::load(et + j), ti = Vec<V>::load(et + half + j);
            const Vec<V> th = Vec<V>::load(rr + j);
            Vec<V> ar, ai;
#pragma unroll
            for (int e = 0; e < V; ++e) {
                float sn, c;
                sincosf(th.v[e], &sn, &c);
                ar.v[e] = hr.v[e] * c - hi.v[e] * sn;
                ai.v[e] = hr.v[e] * sn + hi.v[e] * c;
                const float ur = ar.v[e] - tr.v[e], ui = ai.v[e] - ti.v[e];
                acc += sqrtf(ur * ur + ui * ui);
                if (a.head) {  // the kept side is the tail: t e^{-i theta}
                    ar.v[e] = tr.v[e] * c + ti.v[e] * sn;
                    ai.v[e] = ti.v[e] * c - tr.v[e] * sn;
                }
            }
            if (out && valid) ar.store(out + j), ai.store(out + half + j);  // rotated row, reused downstream
        }
    }

    acc = wave_sum(acc);
    if (a.pos && valid && lane == 0) {
        float s = acc;
        if constexpr (MODEL == KGE_TRANSE || MODEL == KGE_TRANSH || MODEL == KGE_TRANSR)
            s = P == 2 ? sqrtf(acc) : acc;
        if constexpr (MODEL == KGE_ROTATE) s = a.gamma - acc;
        a.pos[b] = s;
    }
}

}  // namespace kge
