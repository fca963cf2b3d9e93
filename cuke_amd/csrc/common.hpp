// Shared device/host helpers for the gfx950 KGE kernels.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/kge_mi355.h"

namespace kge {

constexpr int kWave = 64;

// Launch errors are sticky per host thread: an entry point clears whatever another library left
// behind (KGE_CLEAR_LAUNCH_ERRORS) before its first launch, so that KGE_CHECK_LAUNCH reports only
// this library's own launches.
#define KGE_CLEAR_LAUNCH_ERRORS() ((void)hipGetLastError())
#define KGE_CHECK_LAUNCH()                                   \
    do {                                                     \
        if (hipGetLastError() != hipSuccess) return KGE_ELAUNCH; \
    } while (0)

__host__ __device__ inline int64_t ceil_div(int64_t a, int64_t b) { return (a + b - 1) / b; }

// Butterfly all-reduce over the 64 lanes of a wavefront.
__device__ __forceinline__ float wave_sum(float v)
{
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, kWave);
    return v;
}

__device__ __forceinline__ int wave_sum_i(int v)
{
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, kWave);
    return v;
}

// V consecutive floats moved with one instruction when V == 4 (global_load_dwordx4).
template <int V>
struct Vec;
template <>
struct Vec<4> {
    float v[4];
    __device__ __forceinline__ static Vec load(const float *p)
    {
        const float4 q = *reinterpret_cast<const float4 *>(p);
        return Vec{{q.x, q.y, q.z, q.w}};
    }
    __device__ __forceinline__ void store(float *p) const
    {
        *reinterpret_cast<float4 *>(p) = make_float4(v[0], v[1], v[2], v[3]);
    }
};
template <>
struct Vec<1> {
    float v[1];
    __device__ __forceinline__ static Vec load(const float *p) { return Vec{{*p}}; }
    __device__ __forceinline__ void store(float *p) const { *p = v[0]; }
};

__device__ __forceinline__ float sgn(float x) { return x > 0.0f ? 1.0f : (x < 0.0f ? -1.0f : 0.0f); }

inline bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

inline hipStream_t as_stream(void *s) { return reinterpret_cast<hipStream_t>(s); }

// DistMult / ComplEx pair sums on the vector ALUs instead of the matrix cores (kge_tables.flags)
inline bool pair_sums_valu(const kge_tables *tab) { return (tab->flags & KGE_PAIR_SUMS_VALU) != 0; }

// One entry of the caller's timeline (kge_batch.timeline): the kernel launched last ends here.
inline void timeline_mark(kge_timeline *tl, hipStream_t st, const char *label)
{
    if (!tl || !tl->events || !tl->labels) return;
    if (tl->count < 0 || tl->count >= tl->capacity ||
        hipEventRecord(reinterpret_cast<hipEvent_t>(tl->events[tl->count]), st) != hipSuccess) {
        ++tl->dropped;  // kge_timeline_elapsed refuses a table with holes
        return;
    }
    tl->labels[tl->count++] = label;
}

// floats per relation / auxiliary row for a model with entity width d
inline int64_t rel_width(int model, int64_t d)
{
    return model == KGE_ROTATE ? d / 2 : (model == KGE_RESCAL ? 0 : d);
}
inline int64_t aux_width(int model, int64_t d)
{
    return model == KGE_TRANSH ? d : ((model == KGE_TRANSR || model == KGE_RESCAL) ? d * d : 0);
}

}  // namespace kge
