// The index inspector for up to 65536 ids as device functions, so that its workgroups can run
// either as kernels of their own (inspector.hip) or in front of the workgroups of a score kernel
// in the same launch (FusedInsp below): a digit pass and the dedup have no dependency between
// workgroups, only on the launch before.
#pragma once

#include "common.hpp"

namespace kge {

constexpr int kSortThreads = 256;
constexpr int kMaxDigitBits = 11;
constexpr int kMaxBins = 1 << kMaxDigitBits;

struct Parts {
    const int64_t *p[4];
    int64_t end[4];  // exclusive end offset of each part in the concatenation
    int n_parts;
};

// Key i of the concatenation, with the part table held in registers and the index clamped by the caller: the load
// is unconditional (a branch or a select around a load makes the compiler wait for it on the
// spot, which serialises a batch of loads into one memory round trip each).
struct KeySrc {
    // byte address of key i = base_k + 8 i for the part k that holds position i; the bases are
    // plain integers so that the choice is a per-lane select (choosing among pointer VALUES makes
    // the compiler loop over the distinct pointers of a wave, one waited load per turn)
    uint64_t b0, b1, b2, b3;
    int64_t e0, e1, e2;
    __device__ explicit KeySrc(const Parts &parts)
        : e0(parts.end[0]), e1(parts.end[1]), e2(parts.end[2])
    {
        b0 = reinterpret_cast<uint64_t>(parts.p[0]);
        b1 = reinterpret_cast<uint64_t>(parts.p[1]) - 8u * (uint64_t)e0;
        b2 = reinterpret_cast<uint64_t>(parts.p[2]) - 8u * (uint64_t)e1;
        b3 = reinterpret_cast<uint64_t>(parts.p[3]) - 8u * (uint64_t)e2;
    }
    __device__ __forceinline__ uint32_t operator()(int64_t i) const  // i must be a valid position
    {
        const uint64_t base = i < e0 ? b0 : (i < e1 ? b1 : (i < e2 ? b2 : b3));
        // low word of the int64 id; the address-space-1 pointer makes this a global (not flat) load,
        // which leaves the LDS counter alone so that the histogram atomics need not drain per key
        typedef const uint32_t __attribute__((address_space(1))) *global_u32;
        return *reinterpret_cast<global_u32>(base + 8u * (uint64_t)i);
    }
};

// exclusive scan of s[0..bins) in place (bins <= 2048, 256 threads)
__device__ inline void block_exclusive_scan(uint32_t *s, int bins, uint32_t *wave_tot)
{
    const int per = (bins + kSortThreads - 1) / kSortThreads;  // <= 8
    const int lo = threadIdx.x * per;
    uint32_t loc[kMaxBins / kSortThreads];
    uint32_t sum = 0;
    for (int i = 0; i < per; ++i) {
        const uint32_t v = lo + i < bins ? s[lo + i] : 0;
        loc[i] = sum;
        sum += v;
    }
    // inclusive scan of `sum` across the wave, then across the waves
    const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x >> 6;
    uint32_t inc = sum;
#pragma unroll
    for (int o = 1; o < kWave; o <<= 1) {
        const uint32_t up = __shfl_up(inc, o, kWave);
        if (lane >= o) inc += up;
    }
    if (lane == kWave - 1) wave_tot[wave] = inc;
    __syncthreads();
    uint32_t woff = 0;
    for (int w = 0; w < wave; ++w) woff += wave_tot[w];
    const uint32_t excl = woff + inc - sum;
    for (int i = 0; i < per; ++i)
        if (lo + i < bins) s[lo + i] = excl + loc[i];
    __syncthreads();
}

// ---- small and medium inputs (up to 65536 ids) ---------------------------------------------------
// A workgroup owns 1024 consecutive keys.  The steps of a job are
//   histogram: every workgroup writes the digit histograms of its own keys, one per pass, to the
//              job's workspace (a histogram does not depend on key order, so all passes' bin totals
//              are known before anything is sorted);
//   scatter p: bin starts = column sums of pass p's histograms; the same-digit keys in front of the
//              workgroup come from those histograms too in the first pass, and from a recount of
//              the sorted keys in front of it in a later pass; the workgroup's own keys are ranked
//              stably with wave ballots and scattered.  A job with a single pass is finished here
//              (every non-empty bin is one distinct id);
//   dedup:     run detection over the sorted keys.
// No step depends on another workgroup of the same launch, only on the launch before, so the steps
// run as launches of their own (several index sets sharing them) or as extra workgroups in front
// of another kernel's grid (FusedInsp).
constexpr int kMidThreads = 256;
constexpr int kMidWaves = kMidThreads / kWave;
constexpr int kMidKeys = 1024;  // keys per block: 4 rounds of 64 per wave
constexpr int kMidRounds = kMidKeys / kMidThreads;
constexpr int64_t kMidMaxN = 65536;
constexpr int kMidMaxPass = 3;

struct MidJob {
    Parts parts;
    int64_t n;
    int npass, db;
    kge_inspection out;
    uint32_t *keys_final, *keys_tmp;
    int32_t *vals_tmp;
    uint32_t *hist;  // [kMidMaxPass][workgroups][bins]
};
struct MidJobs {
    MidJob j[4];
};

// Inspector workgroups riding in front of another kernel's grid.  A job with np digit passes
// has np + 2 steps (histogram, np scatters, dedup), one per launch; the four hosts of a
// shared-negative training step are, in order, the per-positive forward kernel, the forward tile
// kernel, the gradient tile kernel and the per-positive gradient kernel (slot 0..3), and a job
// uses the last np + 2 of them (grouped TransR / RESCAL steps: forward GEMM, prep, dX GEMM, dM).
// Workgroup b < blocks belongs to job 0 if b < split, else job 1.
struct FusedInsp {
    MidJob j[2];
    int n_jobs;  // 1 or 2
    int blocks;  // a multiple of 8, so the host's own workgroups keep their XCD (0: nothing fused)
    int split;   // workgroups of job 0
    int slot;
    int lds_bytes;
};

// LDS words a digit pass with `bins` bins needs
// (a job with a single pass also keeps the index of every non-empty bin: one more array)
__host__ __device__ constexpr int mid_pass_lds_words(int bins, int npass)
{
    return (2 + kMidWaves + (npass == 1 ? 1 : 0)) * bins + kMidWaves;
}

// Workgroups of a job, and the per-workgroup digit histograms of pass p in the job's workspace
// (kMidMaxPass tables of [workgroups][bins] counters).
__host__ __device__ inline int mid_blocks(int64_t n) { return n > 0 ? (int)((n + kMidKeys - 1) / kMidKeys) : 1; }
__device__ __forceinline__ uint32_t *mid_hist(const MidJob &J, int pass)
{
    return J.hist + (size_t)pass * mid_blocks(J.n) * (1u << J.db);
}

// Step 0 of a job: the digit histograms of this workgroup's own keys, one per pass (a histogram
// does not depend on the order of the keys, so all passes' totals are known before any sorting).
__host__ __device__ constexpr int mid_hist_lds_words(int bins, int npass) { return bins * npass; }

__device__ __forceinline__ void mid_hist_body(const MidJob &J, int bx, uint32_t *smem)
{
    __builtin_amdgcn_s_setprio(3);  // see mid_scatter_body
    const int n = (int)J.n;
    if (bx * kMidKeys >= n) return;
    const int tid = threadIdx.x;
    const int bins = 1 << J.db;
    const uint32_t mask = (uint32_t)bins - 1;
    const int my0 = bx * kMidKeys;
    const KeySrc src(J.parts);
    uint32_t key[kMidRounds];
#pragma unroll
    for (int j = 0; j < kMidRounds; ++j) {
        const int i = my0 + j * kMidThreads + tid;
        key[j] = src(i < n ? i : n - 1);
    }
    for (int i = tid; i < bins * J.npass; i += kMidThreads) smem[i] = 0;
    __syncthreads();
#pragma unroll
    for (int j = 0; j < kMidRounds; ++j)
        if (my0 + j * kMidThreads + tid < n)
            for (int p = 0; p < J.npass; ++p) atomicAdd(&smem[p * bins + ((key[j] >> (p * J.db)) & mask)], 1u);
    __syncthreads();
    const size_t row = (size_t)bx * bins;
    for (int p = 0; p < J.npass; ++p)
        for (int i = tid; i < bins; i += kMidThreads) mid_hist(J, p)[row + i] = smem[p * bins + i];
}

// One digit pass of job J for the keys [bx * kMidKeys, (bx + 1) * kMidKeys).  Bin starts come from
// the column sums of the per-workgroup histograms (a few coalesced loads per thread).  The number
// of same-digit keys in front of this workgroup comes from the same histograms in the first pass
// (the keys are still in input order, workgroup by workgroup); in a later pass the workgroup counts
// the digits of the sorted keys in front of it itself (batched loads, LDS atomics).  Its own keys
// are ranked stably with wave ballots and scattered.
template <bool FIRST>
__device__ __forceinline__ void mid_scatter_body(const MidJob &J, int pass, int bx, uint32_t *smem)
{
    // The inspection runs next to the score kernels (in front of their workgroups in the same
    // launch, or on its own stream), whose waves fill every SIMD; without a raised wave priority
    // these few workgroups get a fraction of the issue slots.
    __builtin_amdgcn_s_setprio(3);
    const int n = (int)J.n;
    if (pass < 0 || pass >= J.npass || bx * kMidKeys >= n) return;
    const int tid = threadIdx.x, lane = tid & (kWave - 1), wave = tid >> 6;
    const int bins = 1 << J.db;
    uint32_t *s_tot = smem;              // digit totals -> global bin starts
    uint32_t *s_bef = smem + bins;       // same digit, earlier workgroups
    uint32_t *s_cnt = smem + 2 * bins;   // [kMidWaves][bins] per-wave running counts
    uint32_t *s_w = smem + (2 + kMidWaves) * bins;
    const uint32_t mask = (uint32_t)bins - 1;
    const int shift = pass * J.db;
    const bool to_final = ((J.npass - 1 - pass) & 1) == 0;
    const uint32_t *kin = to_final ? J.keys_tmp : J.keys_final;  // (unused in the first pass)
    const int32_t *vin = to_final ? J.vals_tmp : J.out.perm;
    uint32_t *kout = to_final ? J.keys_final : J.keys_tmp;
    int32_t *vout = to_final ? J.out.perm : J.vals_tmp;
    const int my0 = bx * kMidKeys;

    // own keys first (their loads overlap the histogram reads); positions past n are clamped and
    // masked at their use
    const KeySrc src(J.parts);
    const int last = n - 1;
    uint32_t key[kMidRounds];
    int32_t val[kMidRounds];
#pragma unroll
    for (int j = 0; j < kMidRounds; ++j) {
        const int i = my0 + wave * (kMidRounds * kWave) + j * kWave + lane;
        const int ic = i < n ? i : last;
        if constexpr (FIRST) key[j] = src(ic), val[j] = i;
        else key[j] = kin[ic], val[j] = vin[ic];
    }
    // column sums of the histograms: all workgroups, and those before this one.  A thread takes
    // four consecutive bins with one 128-bit load per row, sixteen rows in flight.
    const uint4 *H = reinterpret_cast<const uint4 *>(mid_hist(J, pass));
    const int nblk = mid_blocks(n), quads = bins >> 2;  // bins >= 4
    for (int q = tid; q < quads; q += kMidThreads) {
        uint4 tot = make_uint4(0, 0, 0, 0), bef = make_uint4(0, 0, 0, 0);
        constexpr int kFly = 16;
        for (int b0 = 0; b0 < nblk; b0 += kFly) {
            uint4 v[kFly];
#pragma unroll
            for (int u = 0; u < kFly; ++u) {
                const int b = b0 + u < nblk ? b0 + u : nblk - 1;  // clamped: unconditional loads, masked below
                v[u] = H[(size_t)b * quads + q];
            }
#pragma unroll
            for (int u = 0; u < kFly; ++u) {
                const uint32_t in = b0 + u < nblk ? ~0u : 0u, pre = b0 + u < bx ? ~0u : 0u;
                tot.x += v[u].x & in, tot.y += v[u].y & in, tot.z += v[u].z & in, tot.w += v[u].w & in;
                bef.x += v[u].x & pre, bef.y += v[u].y & pre, bef.z += v[u].z & pre, bef.w += v[u].w & pre;
            }
        }
        reinterpret_cast<uint4 *>(s_tot)[q] = tot;
        reinterpret_cast<uint4 *>(s_bef)[q] = bef;
#pragma unroll
        for (int w = 0; w < kMidWaves; ++w) reinterpret_cast<uint4 *>(s_cnt + w * bins)[q] = make_uint4(0, 0, 0, 0);
    }
    __syncthreads();
    if (pass > 0) {  // s_bef held the histogram-order count, which only the first pass can use
        for (int i = tid; i < bins; i += kMidThreads) s_bef[i] = 0;
        __syncthreads();
        // (my0 is a multiple of 1024 and the key buffers are 256-byte aligned: whole groups of four
        // keys per 128-bit load, sixteen groups per thread in flight)
        constexpr int kBatch = 16;
        const uint4 *kin4 = reinterpret_cast<const uint4 *>(kin);
        const int groups = my0 >> 2;
        for (int g0 = 0; g0 < groups; g0 += kBatch * kMidThreads) {
            uint4 kb[kBatch];
#pragma unroll
            for (int u = 0; u < kBatch; ++u) {
                const int g = g0 + u * kMidThreads + tid;
                kb[u] = kin4[g < groups ? g : groups - 1];  // clamped: unconditional loads, masked below
            }
#pragma unroll
            for (int u = 0; u < kBatch; ++u)
                if (g0 + u * kMidThreads + tid < groups) {
                    atomicAdd(&s_bef[(kb[u].x >> shift) & mask], 1u);
                    atomicAdd(&s_bef[(kb[u].y >> shift) & mask], 1u);
                    atomicAdd(&s_bef[(kb[u].z >> shift) & mask], 1u);
                    atomicAdd(&s_bef[(kb[u].w >> shift) & mask], 1u);
                }
        }
        __syncthreads();
    }
    // A job with a single pass sorts by the whole key, so every non-empty bin is one distinct id:
    // the run structure falls out of the histogram and no dedup step is needed.
    const bool finish = J.npass == 1;
    uint32_t *s_u = s_w + kMidWaves;  // finish: number of non-empty bins below this one
    uint32_t nonempty = 0, n_unique = 0;  // bit u of nonempty: bin tid + 256 u has keys
    if (finish) {
        for (int u = 0, bin = tid; bin < bins; ++u, bin += kMidThreads) {
            const uint32_t f = s_tot[bin] > 0 ? 1u : 0u;
            nonempty |= f << u;
            s_u[bin] = f;
        }
        __syncthreads();
        block_exclusive_scan(s_u, bins, s_w);
        n_unique = s_u[bins - 1] + (s_tot[bins - 1] > 0 ? 1u : 0u);
    }
    block_exclusive_scan(s_tot, bins, s_w);  // s_tot[bin] = first position of the bin
    if (finish && bx == 0) {
        for (int u = 0, bin = tid; bin < bins; ++u, bin += kMidThreads)
            if ((nonempty >> u) & 1u) {
                J.out.unique_ids[s_u[bin]] = (int64_t)bin;
                J.out.seg_offsets[s_u[bin]] = (int32_t)s_tot[bin];
            }
        if (tid == 0) {
            J.out.num_unique[0] = (int32_t)n_unique;
            J.out.seg_offsets[n_unique] = n;
        }
    }

    const uint64_t lt_mask = lane ? (~0ull >> (kWave - lane)) : 0ull;
    uint32_t lrank[kMidRounds];
#pragma unroll
    for (int j = 0; j < kMidRounds; ++j) {
        const int i = my0 + wave * (kMidRounds * kWave) + j * kWave + lane;
        const bool ok = i < n;
        const uint32_t dg = (key[j] >> shift) & mask;
        uint64_t peers = __ballot(ok);
        for (int bit = 0; bit < J.db; ++bit) {
            const bool one = (dg >> bit) & 1u;
            const uint64_t mm = __ballot(one);
            peers &= one ? mm : ~mm;
        }
        const int leader = __ffsll((unsigned long long)peers) - 1;
        uint32_t old = 0;
        if (ok && lane == leader) {
            old = s_cnt[wave * bins + dg];
            s_cnt[wave * bins + dg] = old + __popcll(peers);
        }
        old = __shfl(old, leader < 0 ? 0 : leader, kWave);
        lrank[j] = old + __popcll(peers & lt_mask);
        __builtin_amdgcn_wave_barrier();
    }
    __syncthreads();
    for (int bin = tid; bin < bins; bin += kMidThreads) {
        uint32_t run = s_tot[bin] + s_bef[bin];
#pragma unroll
        for (int w = 0; w < kMidWaves; ++w) {
            const uint32_t c = s_cnt[w * bins + bin];
            s_cnt[w * bins + bin] = run;
            run += c;
        }
    }
    __syncthreads();
#pragma unroll
    for (int j = 0; j < kMidRounds; ++j) {
        const int i = my0 + wave * (kMidRounds * kWave) + j * kWave + lane;
        if (i < n) {
            const uint32_t dg = (key[j] >> shift) & mask;
            const uint32_t pos = s_cnt[wave * bins + dg] + lrank[j];
            kout[pos] = key[j];
            vout[pos] = val[j];
            if (finish) {
                J.out.sorted_seg[pos] = (int32_t)s_u[dg];
                J.out.inverse[val[j]] = (int32_t)s_u[dg];
            }
        }
    }
}

constexpr int kMidDedupLdsWords = 2 * kMidWaves;

// Run detection over the sorted keys [bx * kMidKeys, (bx + 1) * kMidKeys) of job J.
__device__ __forceinline__ void mid_dedup_body(const MidJob &J, int bx, uint32_t *smem)
{
    uint32_t *s_red = smem, *s_scan = smem + kMidWaves;
    __builtin_amdgcn_s_setprio(3);
    const int n = (int)J.n;
    const int nblk = n > 0 ? (n + kMidKeys - 1) / kMidKeys : 1;
    if (bx >= nblk || (J.npass == 1 && n > 0)) return;  // single pass: finished by the scatter step
    const int tid = threadIdx.x, lane = tid & (kWave - 1), wave = tid >> 6;
    const uint32_t *keys = J.keys_final;
    const int my0 = bx * kMidKeys;
    // run heads before this block
    // (my0 is a multiple of 1024: every thread takes whole groups of four keys with one 128-bit
    // load, plus the key in front of the group; eight groups in flight)
    uint32_t before = 0;
    for (int g0 = 0; g0 < my0 / 4; g0 += 8 * kMidThreads) {
        uint4 q[8];
        uint32_t pv[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            const int g = g0 + u * kMidThreads + tid;
            const int gc = g < my0 / 4 ? g : my0 / 4 - 1;  // clamped: unconditional loads, masked below
            q[u] = reinterpret_cast<const uint4 *>(keys)[gc];
            pv[u] = keys[gc > 0 ? 4 * gc - 1 : 0];
        }
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            const int g = g0 + u * kMidThreads + tid;
            if (g < my0 / 4)
                before += ((g == 0 || q[u].x != pv[u]) ? 1 : 0) + (q[u].y != q[u].x ? 1 : 0) +
                          (q[u].z != q[u].y ? 1 : 0) + (q[u].w != q[u].z ? 1 : 0);
        }
    }
    before = (uint32_t)wave_sum_i((int)before);
    if (lane == 0) s_red[wave] = before;
    // thread owns 4 consecutive sorted positions
    const int lo = my0 + tid * kMidRounds;
    uint32_t k[kMidRounds];
    bool head[kMidRounds];
    uint32_t mine = 0;
    uint32_t prev = (lo > 0 && lo < n) ? keys[lo - 1] : 0;
#pragma unroll
    for (int j = 0; j < kMidRounds; ++j) {
        const int i = lo + j;
        k[j] = i < n ? keys[i] : 0;
        head[j] = i < n && (i == 0 || k[j] != prev);
        prev = k[j];
        mine += head[j] ? 1 : 0;
    }
    uint32_t inc = mine;
#pragma unroll
    for (int o = 1; o < kWave; o <<= 1) {
        const uint32_t up = __shfl_up(inc, o, kWave);
        if (lane >= o) inc += up;
    }
    if (lane == kWave - 1) s_scan[wave] = inc;
    __syncthreads();
    before = 0;
    uint32_t here = 0;
    for (int w = 0; w < kMidWaves; ++w) before += s_red[w], here += s_scan[w];
    uint32_t run = before + inc - mine;
    for (int w = 0; w < wave; ++w) run += s_scan[w];
    if (bx == nblk - 1 && tid == 0) {
        J.out.num_unique[0] = (int32_t)(before + here);
        J.out.seg_offsets[before + here] = n;
    }
#pragma unroll
    for (int j = 0; j < kMidRounds; ++j) {
        const int i = lo + j;
        if (i < n) {
            if (head[j]) {
                J.out.unique_ids[run] = (int64_t)k[j];
                J.out.seg_offsets[run] = i;
                ++run;
            }
            const int32_t seg = (int32_t)run - 1;
            J.out.sorted_seg[i] = seg;
            J.out.inverse[J.out.perm[i]] = seg;
        }
    }
}


constexpr int kFusedSlots = 4;

// Called first thing by a host kernel; true = this workgroup was an inspector workgroup and is done.
__device__ __forceinline__ bool fused_insp_block(const FusedInsp &f, uint32_t *smem)
{
    const int b = blockIdx.x;
    if (b >= f.blocks) return false;
    if (b >= f.split && f.n_jobs < 2) return true;  // padding up to a multiple of 8 workgroups
    const MidJob &J = f.j[b < f.split ? 0 : 1];
    const int bx = b < f.split ? b : b - f.split;
    const int step = f.slot - (kFusedSlots - 2 - J.npass);  // 0: histogram, 1..np: scatter, np + 1: dedup
    if (step == 0) mid_hist_body(J, bx, smem);
    else if (step == 1) mid_scatter_body<true>(J, 0, bx, smem);
    else if (step > 1 && step <= J.npass) mid_scatter_body<false>(J, step - 1, bx, smem);
    else if (step == J.npass + 1) mid_dedup_body(J, bx, smem);
    return true;
}

// host side (inspector.hip): fills `out` for one slot from one or two inspection jobs;
// KGE_EUNSUPPORTED when a job is too large or its table needs more than two digit passes of
// kMaxDigitBits bits
int plan_fused_inspection(const kge_inspect_job *jobs, int n_jobs, int slot, FusedInsp *out);

// Jobs that ride with a model's kernels: both index sets with the shared-negative kernels, the
// entity set alone with the grouped TransR / RESCAL kernels (their relation groups must exist
// before the forward pass starts).
inline int fused_job_count(int model) { return model == KGE_TRANSR || model == KGE_RESCAL ? 1 : 2; }

}  // namespace kge
