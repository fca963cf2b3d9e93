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
    // One launch instead of two: seg_ticket_ints(n, d) counters, ALL ZERO when the reduction starts
    // (a kernel in front of it on the stream clears them, see ZeroRider; the reduction leaves them zero
    // again).  The wave that completes a run crossing block boundaries last adds up its partial rows.
    // Null: level 2 runs as a launch of its own.
    int32_t *tickets = nullptr;
    // Optional transform of the rows as they are loaded: row i counts as scale[i] * phi(occ[i]) with
    // scale[i] = num[i] (den null) or num[i] / den[i] (0 where den[i] <= 0) and phi = sign or identity.
    // Lets a consumer sum rows that only exist as "coefficient times another array's row" without a
    // kernel that writes them out first.  scaled with num null: the rows count as zero.
    bool scaled = false, sign_rows = false;
    const float *scale_num = nullptr, *scale_den = nullptr;
};

inline int64_t seg_partial_floats(int64_t n, int64_t d) { return ceil_div(n > 0 ? n : 1, kSegL) * 2 * d; }
inline int64_t seg_ticket_ints(int64_t n, int64_t d) { return ceil_div(n > 0 ? n : 1, kSegL) * ceil_div(d > 0 ? d : 1, kWave); }

// Words that a kernel clears on behalf of a later kernel of the same call (the reduction's tickets):
// its first workgroups stride over them before they turn to their own work.
struct ZeroRider {
    int32_t *p = nullptr;
    int64_t n = 0;
};
#if defined(__HIPCC__)
__device__ __forceinline__ void zero_rider(const ZeroRider &z)
{
    const int nb = gridDim.x < 8 ? (int)gridDim.x : 8;
    if (z.n > 0 && (int)blockIdx.x < nb && blockIdx.y == 0)
        for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < z.n; i += (int64_t)nb * blockDim.x) z.p[i] = 0;
}
#endif

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
