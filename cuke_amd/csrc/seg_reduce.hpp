// Segmented reduction of per-occurrence gradient rows into one row per distinct id.
#pragma once

#include "common.hpp"

namespace kge {

constexpr int kSegL = 8;  // sorted positions per level-1 wave

struct SegJob {
    const float *occ;            // [n, d] occurrence rows
    const kge_inspection *ins;   // sorted order / runs of the ids the rows belong to
    int d;
    float *out;                  // [U, d]
    float *partial;              // seg_partial_floats(n, d) floats of scratch
    bool identity_perm;          // occ is already stored in sorted order
    // Optional transform of the rows as they are loaded: row i counts as scale[i] * phi(occ[i]) with
    // scale[i] = num[i] (den null) or num[i] / den[i] (0 where den[i] <= 0) and phi = sign or identity.
    // Lets a consumer sum rows that only exist as "coefficient times another array's row" without a
    // kernel that writes them out first.  scaled with num null: the rows count as zero.
    bool scaled = false, sign_rows = false;
    const float *scale_num = nullptr, *scale_den = nullptr;
    // wrap > 0: occurrence i >= wrap takes row i - wrap (and its scale) with the opposite sign: the head and tail
    // occurrences of a translation model's triple share one row, +row for the head and -row for the tail.
    int64_t wrap = 0;
};

inline int64_t seg_partial_floats(int64_t n, int64_t d) { return ceil_div(n > 0 ? n : 1, kSegL) * 2 * d; }

// Work that depends on nothing the reduction produces and rides in its level-1 launch (one more
// slice of the grid): out row seg[i] = part row first[i] + ... + part row first[i] + cnt[i] - 1, for
// i < num[0] (all four arrays live on the device).  TransR's split relation groups finish their
// projection gradients this way instead of in a launch of their own.
struct SumRider {
    const float *part = nullptr;
    float *out = nullptr;
    const int32_t *num = nullptr, *seg = nullptr, *first = nullptr, *cnt = nullptr;
    int64_t row_floats = 0;  // a multiple of 4
    int max_sums = 0;        // 0: no rider
};

struct SegArgs {
    const float *occ;
    const int32_t *perm, *sorted_seg, *seg_offsets;
    int64_t n;
    int d;
    float *out, *partial;
    const float *scale_num, *scale_den;   // row transform (SegJob), transform bit 0 = scaled, bit 1 = sign
    int transform;
    int wrap;                             // SegJob::wrap (0: none)
};
struct SegArgs3 {
    SegArgs j[3];
};


// The level-1 pass of up to three jobs as extra workgroups at the end of another kernel's grid: a pass that
// does not depend on that kernel (only on launches before it) runs in its shadow instead of in a launch of its
// own.  plan_seg_l1_rider() fills it on the host; the carrying kernel appends blocks() workgroups and calls
// seg_l1_rider_block() with the workgroup's index among them.
struct SegL1Rider {
    SegArgs3 jobs;
    int n_jobs = 0, blocks_x = 0, v4 = 0;
    int blocks() const { return n_jobs * blocks_x; }
};
SegL1Rider plan_seg_l1_rider(const SegJob *jobs, int n_jobs);

// Up to three jobs share the same two launches.  level1_rode: the level-1 pass of exactly these jobs has run as a
// SegL1Rider; only level 2 is launched, and it carries the rider's sums.
int launch_seg_reduce_jobs(const SegJob *jobs, int n_jobs, hipStream_t st, kge_timeline *timeline = nullptr,
                           const SumRider *rider = nullptr, bool level1_rode = false);

#ifdef __HIPCC__
// Level 1 for wave `w` of job `a` (a wave owns kSegL consecutive sorted positions and one chunk of 64 V columns).
// Uses no LDS, so the workgroups of a level-1 pass can also ride at the end of another kernel's grid (SegL1Rider).
template <int V>
__device__ __forceinline__ void seg_l1_wave(const SegArgs &a, int64_t w)
{
    const int lane = threadIdx.x & (kWave - 1);
    const int d = a.d;
    const int nch = (d + kWave * V - 1) / (kWave * V);
    const int64_t j = w / nch;
    const int colv = (int)(w % nch) * kWave * V + lane * V;
    const int64_t p0 = j * kSegL;
    if (p0 >= a.n) return;
    const int cnt = (int)((a.n - p0) < kSegL ? (a.n - p0) : kSegL);
    const bool active = colv < d;

    // Everything the walk needs is loaded up front in batches of unconditional loads (positions
    // past the end re-read the last valid one, an inactive lane reads column 0, both are masked
    // afterwards): a branch or a select around a load would make the compiler wait for each load
    // on the spot and turn the eight rows into eight serial round trips.
    int64_t pc[kSegL];
#pragma unroll
    for (int q = 0; q < kSegL; ++q) pc[q] = p0 + (q < cnt ? q : cnt - 1);
    int src[kSegL], seg[kSegL];
    if (a.perm) {  // uniform
#pragma unroll
        for (int q = 0; q < kSegL; ++q) src[q] = a.perm[pc[q]];
    } else {
#pragma unroll
        for (int q = 0; q < kSegL; ++q) src[q] = (int)pc[q];
    }
#pragma unroll
    for (int q = 0; q < kSegL; ++q) seg[q] = a.sorted_seg[pc[q]];
    float wsign[kSegL];
#pragma unroll
    for (int q = 0; q < kSegL; ++q) {
        const bool second = a.wrap > 0 && src[q] >= a.wrap;
        wsign[q] = second ? -1.0f : 1.0f;
        src[q] = second ? src[q] - a.wrap : src[q];
    }
    const int cc = active ? colv : 0;
    Vec<V> v[kSegL];
#pragma unroll
    for (int q = 0; q < kSegL; ++q) v[q] = Vec<V>::load(a.occ + (int64_t)src[q] * d + cc);
    if (a.transform) {  // uniform: the rows count as scale * phi(row)
        float sc[kSegL];
#pragma unroll
        for (int q = 0; q < kSegL; ++q) sc[q] = (a.transform & 1) ? (a.scale_num ? a.scale_num[src[q]] : 0.0f) : 1.0f;
        if ((a.transform & 1) && a.scale_den) {
            float den[kSegL];
#pragma unroll
            for (int q = 0; q < kSegL; ++q) den[q] = a.scale_den[src[q]];
#pragma unroll
            for (int q = 0; q < kSegL; ++q) sc[q] = den[q] > 0.0f ? sc[q] / den[q] : 0.0f;
        }
#pragma unroll
        for (int q = 0; q < kSegL; ++q)
#pragma unroll
            for (int e = 0; e < V; ++e) v[q].v[e] = wsign[q] * (sc[q] * ((a.transform & 2) ? sgn(v[q].v[e]) : v[q].v[e]));
    } else if (a.wrap > 0) {
#pragma unroll
        for (int q = 0; q < kSegL; ++q)
#pragma unroll
            for (int e = 0; e < V; ++e) v[q].v[e] *= wsign[q];
    }
    // A run starts before this block iff it shares its id with the position in front of the block,
    // and runs on past it iff it shares it with the position behind: two loads instead of the run
    // bounds of every position.
    const int seg_before = a.sorted_seg[p0 > 0 ? p0 - 1 : 0], seg_after = a.sorted_seg[p0 + cnt < a.n ? p0 + cnt : p0];
    const int prev_id = p0 > 0 ? seg_before : -1;
    const int next_id = p0 + cnt < a.n ? seg_after : -1;

    Vec<V> acc;
#pragma unroll
    for (int e = 0; e < V; ++e) acc.v[e] = 0.0f;
    auto flush = [&](int sg) {
        float *dst;
        if (sg == prev_id) dst = a.partial + (j * 2 + 0) * (int64_t)d;       // began in an earlier block
        else if (sg == next_id) dst = a.partial + (j * 2 + 1) * (int64_t)d;  // continues in a later block
        else dst = a.out + (int64_t)sg * d;                                   // wholly inside: final
        if (active) acc.store(dst + colv);
    };
#pragma unroll
    for (int q = 0; q < kSegL; ++q) {
        if (q < cnt) {
            if (q > 0 && seg[q] != seg[q - 1]) {
                flush(seg[q - 1]);
#pragma unroll
                for (int e = 0; e < V; ++e) acc.v[e] = 0.0f;
            }
#pragma unroll
            for (int e = 0; e < V; ++e) acc.v[e] += v[q].v[e];
        }
    }
    flush(seg[cnt - 1]);
}


__device__ __forceinline__ void seg_l1_rider_block(const SegL1Rider &r, int rb)
{
    const int slice = rb / r.blocks_x;
    const int64_t w = (int64_t)(rb % r.blocks_x) * 4 + (threadIdx.x >> 6);
    if (r.v4) seg_l1_wave<4>(r.jobs.j[slice], w);
    else seg_l1_wave<1>(r.jobs.j[slice], w);
}
#endif

}  // namespace kge
