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

// Up to three jobs share the same two launches.
int launch_seg_reduce_jobs(const SegJob *jobs, int n_jobs, hipStream_t st, kge_timeline *timeline = nullptr,
                           const SumRider *rider = nullptr);

}  // namespace kge
