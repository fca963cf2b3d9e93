// GPU index inspector: stable LSD radix sort of (id, position) pairs followed by
// run detection, giving unique rows, segment offsets, the sort permutation and the
// inverse map.  It stands where the reference runs its per-16 bitonic inspector
// (apps/kge/inspection/inspector.cu:68-136, called from apps/kge/kge.py:249-271) but
// produces the whole-batch structure the gather and segmented-reduction kernels use.
//
// Keys are the low 32 bits of the ids (tables have < 2^32 rows); only as many digit
// passes are run as the table's row count needs.  Every pass is: per-block digit
// histogram -> column scan -> stable scatter.  Stability inside a block comes from
// wave-level peer matching (ballots), not from atomics, so the result is
// deterministic and equals a stable argsort.
#include "inspector_mid.hpp"

namespace kge {

constexpr int kSortWaves = kSortThreads / kWave;
constexpr int kKeysPerThread = 8;
constexpr int kKeysPerBlock = kSortThreads * kKeysPerThread;  // 2048
constexpr int kFusedScanBlocks = 32;  // up to this many blocks the scatter kernel scans the
                                      // histogram columns itself (one launch less per pass)

// ---- pass step 1: per-block digit histogram --------------------------------------------
__global__ __launch_bounds__(kSortThreads) void radix_hist_kernel(Parts parts, const uint32_t *keys_in,
                                                                  int64_t n, int shift, int bins,
                                                                  uint32_t *hist)
{
    __builtin_amdgcn_s_setprio(3);  // see inspect_mid_pass_kernel
    __shared__ uint32_t sh[kMaxBins];
    for (int i = threadIdx.x; i < bins; i += kSortThreads) sh[i] = 0;
    __syncthreads();
    const int64_t base = (int64_t)blockIdx.x * kKeysPerBlock;
    const uint32_t mask = (uint32_t)bins - 1;
    // all loads first (clamped, unconditional), then the counting
    const KeySrc src(parts);
    uint32_t kb[kKeysPerThread];
    if (keys_in) {  // uniform
#pragma unroll
        for (int j = 0; j < kKeysPerThread; ++j) {
            const int64_t i = base + j * kSortThreads + threadIdx.x;
            kb[j] = keys_in[i < n ? i : n - 1];
        }
    } else {
#pragma unroll
        for (int j = 0; j < kKeysPerThread; ++j) {
            const int64_t i = base + j * kSortThreads + threadIdx.x;
            kb[j] = src(i < n ? i : n - 1);
        }
    }
#pragma unroll
    for (int j = 0; j < kKeysPerThread; ++j)
        if (base + j * kSortThreads + threadIdx.x < n) atomicAdd(&sh[(kb[j] >> shift) & mask], 1u);
    __syncthreads();
    for (int i = threadIdx.x; i < bins; i += kSortThreads) hist[(int64_t)blockIdx.x * bins + i] = sh[i];
}

// ---- pass step 2 (many blocks only): exclusive scan down each histogram column ---------
__global__ void radix_colscan_kernel(uint32_t *hist, uint32_t *totals, int bins, int nblocks)
{
    __builtin_amdgcn_s_setprio(3);  // see inspect_mid_pass_kernel
    const int bin = blockIdx.x * blockDim.x + threadIdx.x;
    if (bin >= bins) return;
    uint32_t run = 0;
    for (int b = 0; b < nblocks; ++b) {
        const uint32_t v = hist[(int64_t)b * bins + bin];
        hist[(int64_t)b * bins + bin] = run;
        run += v;
    }
    totals[bin] = run;
}

// ---- pass step 3: stable scatter ---------------------------------------------------------
__global__ __launch_bounds__(kSortThreads) void radix_scatter_kernel(
    Parts parts, const uint32_t *keys_in, const int32_t *vals_in, int64_t n, int shift, int digit_bits,
    const uint32_t *hist, const uint32_t *totals, int nblocks, int fused_scan, uint32_t *keys_out,
    int32_t *vals_out)
{
    __builtin_amdgcn_s_setprio(3);  // see inspect_mid_pass_kernel
    __shared__ uint32_t s_base[kMaxBins];               // global start of (bin, this block)
    __shared__ uint32_t s_cnt[kSortWaves][kMaxBins];    // per-wave running digit counts
    __shared__ uint32_t s_wtot[kSortWaves];
    const int bins = 1 << digit_bits;
    const uint32_t mask = (uint32_t)bins - 1;
    const int tid = threadIdx.x, lane = tid & (kWave - 1), wave = tid >> 6;
    const int me = blockIdx.x;

    // bin totals -> s_base (scanned below); this block's offset inside each bin -> s_cnt[0] (temp)
    for (int bin = tid; bin < bins; bin += kSortThreads) {
        uint32_t tot, part;
        if (fused_scan) {
            tot = 0, part = 0;
            for (int b = 0; b < nblocks; ++b) {
                const uint32_t v = hist[(int64_t)b * bins + bin];
                tot += v;
                part += b < me ? v : 0;
            }
        } else {
            tot = totals[bin];
            part = hist[(int64_t)me * bins + bin];
        }
        s_base[bin] = tot;
        s_cnt[0][bin] = part;
    }
    __syncthreads();
    block_exclusive_scan(s_base, bins, s_wtot);
    for (int bin = tid; bin < bins; bin += kSortThreads) {
        s_base[bin] += s_cnt[0][bin];
    }
    __syncthreads();
    for (int bin = tid; bin < bins; bin += kSortThreads)
#pragma unroll
        for (int w = 0; w < kSortWaves; ++w) s_cnt[w][bin] = 0;
    __syncthreads();

    // each wave ranks its 512 consecutive keys in 8 rounds of 64, in order
    const int64_t wbase = (int64_t)me * kKeysPerBlock + (int64_t)wave * (kKeysPerThread * kWave);
    uint32_t key[kKeysPerThread], lrank[kKeysPerThread];
    int32_t val[kKeysPerThread];
    const uint64_t lt_mask = lane ? (~0ull >> (kWave - lane)) : 0ull;
    {  // all key / value loads of the thread in one batch (clamped, unconditional)
        const KeySrc src(parts);
        if (keys_in) {  // uniform: later passes read the previous pass's output
#pragma unroll
            for (int j = 0; j < kKeysPerThread; ++j) {
                const int64_t i = wbase + j * kWave + lane;
                const int64_t ic = i < n ? i : n - 1;
                key[j] = keys_in[ic], val[j] = vals_in[ic];
            }
        } else {
#pragma unroll
            for (int j = 0; j < kKeysPerThread; ++j) {
                const int64_t i = wbase + j * kWave + lane;
                key[j] = src(i < n ? i : n - 1), val[j] = (int32_t)i;
            }
        }
    }
#pragma unroll
    for (int j = 0; j < kKeysPerThread; ++j) {
        const int64_t i = wbase + j * kWave + lane;
        const bool ok = i < n;
        const uint32_t dg = (key[j] >> shift) & mask;
        uint64_t peers = __ballot(ok);
        for (int bit = 0; bit < digit_bits; ++bit) {
            const bool one = (dg >> bit) & 1u;
            const uint64_t m = __ballot(one);
            peers &= one ? m : ~m;
        }
        // lanes with !ok fall out: their `peers` may be anything but they never write
        const int leader = __ffsll((unsigned long long)peers) - 1;
        const uint32_t cnt = __popcll(peers);
        uint32_t old = 0;
        if (ok && lane == leader) {
            old = s_cnt[wave][dg];
            s_cnt[wave][dg] = old + cnt;
        }
        old = __shfl(old, leader < 0 ? 0 : leader, kWave);
        lrank[j] = old + __popcll(peers & lt_mask);
        __builtin_amdgcn_wave_barrier();  // keep the rounds' LDS counter updates in order
    }
    __syncthreads();
    // turn per-wave counts into per-wave start positions
    for (int bin = tid; bin < bins; bin += kSortThreads) {
        uint32_t run = s_base[bin];
#pragma unroll
        for (int w = 0; w < kSortWaves; ++w) {
            const uint32_t c = s_cnt[w][bin];
            s_cnt[w][bin] = run;
            run += c;
        }
    }
    __syncthreads();
#pragma unroll
    for (int j = 0; j < kKeysPerThread; ++j) {
        const int64_t i = wbase + j * kWave + lane;
        if (i < n) {
            const uint32_t dg = (key[j] >> shift) & mask;
            const uint32_t pos = s_cnt[wave][dg] + lrank[j];
            keys_out[pos] = key[j];
            vals_out[pos] = val[j];
        }
    }
}

// ---- dedup -------------------------------------------------------------------------------
__global__ __launch_bounds__(kSortThreads) void count_heads_kernel(const uint32_t *keys, int64_t n,
                                                                   uint32_t *block_heads)
{
    __builtin_amdgcn_s_setprio(3);  // see inspect_mid_pass_kernel
    __shared__ uint32_t s_w[kSortWaves];
    const int64_t base = (int64_t)blockIdx.x * kKeysPerBlock;
    int c = 0;
#pragma unroll
    for (int j = 0; j < kKeysPerThread; ++j) {
        const int64_t i = base + j * kSortThreads + threadIdx.x;
        if (i < n) c += (i == 0 || keys[i] != keys[i - 1]) ? 1 : 0;
    }
    c = wave_sum_i(c);
    if ((threadIdx.x & (kWave - 1)) == 0) s_w[threadIdx.x >> 6] = (uint32_t)c;
    __syncthreads();
    if (threadIdx.x == 0) {
        uint32_t t = 0;
        for (int w = 0; w < kSortWaves; ++w) t += s_w[w];
        block_heads[blockIdx.x] = t;
    }
}

__global__ __launch_bounds__(kSortThreads) void finalize_kernel(const uint32_t *keys, const int32_t *perm,
                                                                int64_t n, const uint32_t *block_heads,
                                                                int nblocks, kge_inspection out)
{
    __builtin_amdgcn_s_setprio(3);  // see inspect_mid_pass_kernel
    __shared__ uint32_t s_red[kSortWaves], s_all[kSortWaves], s_scan[kSortWaves];
    const int tid = threadIdx.x, lane = tid & (kWave - 1), wave = tid >> 6;
    const int me = blockIdx.x;
    // heads in the blocks before this one, and in all blocks
    uint32_t before = 0, all = 0;
    for (int b = tid; b < nblocks; b += kSortThreads) {
        const uint32_t v = block_heads[b];
        all += v;
        before += b < me ? v : 0;
    }
    before = (uint32_t)wave_sum_i((int)before);
    all = (uint32_t)wave_sum_i((int)all);
    if (lane == 0) s_red[wave] = before, s_all[wave] = all;
    __syncthreads();
    before = 0, all = 0;
    for (int w = 0; w < kSortWaves; ++w) before += s_red[w], all += s_all[w];
    if (me == 0 && tid == 0) {
        out.num_unique[0] = (int32_t)all;
        out.seg_offsets[all] = (int32_t)n;
    }
    // thread owns 8 consecutive positions so that a plain running sum gives the ranks
    const int64_t lo = (int64_t)me * kKeysPerBlock + (int64_t)tid * kKeysPerThread;
    uint32_t k[kKeysPerThread];
    bool head[kKeysPerThread];
    uint32_t mine = 0;
    uint32_t prev = (lo > 0 && lo < n) ? keys[lo - 1] : 0;
#pragma unroll
    for (int j = 0; j < kKeysPerThread; ++j) {
        const int64_t i = lo + j;
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
    uint32_t run = before + inc - mine;
    for (int w = 0; w < wave; ++w) run += s_scan[w];
#pragma unroll
    for (int j = 0; j < kKeysPerThread; ++j) {
        const int64_t i = lo + j;
        if (i >= n) break;
        if (head[j]) {
            out.unique_ids[run] = (int64_t)k[j];
            out.seg_offsets[run] = (int32_t)i;
            ++run;
        }
        const int32_t seg = (int32_t)run - 1;
        out.sorted_seg[i] = seg;
        out.inverse[perm[i]] = seg;
    }
}

// ---- small and medium inputs: the mid-path bodies as kernels of their own -------------------
__global__ __launch_bounds__(kMidThreads) void inspect_mid_hist_kernel(MidJobs jobs)
{
    __shared__ uint32_t smem[mid_hist_lds_words(kMaxBins, kMidMaxPass)];
    mid_hist_body(jobs.j[blockIdx.y], blockIdx.x, smem);
}

template <bool FIRST>
__global__ __launch_bounds__(kMidThreads) void inspect_mid_scatter_kernel(MidJobs jobs, int pass)
{
    __shared__ uint32_t smem[mid_pass_lds_words(kMaxBins, 1)];
    mid_scatter_body<FIRST>(jobs.j[blockIdx.y], pass, blockIdx.x, smem);
}

__global__ __launch_bounds__(kMidThreads) void inspect_mid_dedup_kernel(MidJobs jobs)
{
    __shared__ uint32_t smem[kMidDedupLdsWords];
    mid_dedup_body(jobs.j[blockIdx.y], blockIdx.x, smem);
}

// ---- host side ---------------------------------------------------------------------------
struct SortPlan {
    int bits, npass, digit_bits;
    int64_t nblocks;
    size_t off_keys0, off_keys1, off_vals, off_hist, off_totals, off_heads, total;
};

static size_t align_up(size_t x) { return (x + 255) & ~size_t(255); }

static int key_bits(int64_t n_rows)
{
    int bits = 1;
    while (bits < 32 && (int64_t(1) << bits) < n_rows) ++bits;
    return bits;
}

static SortPlan make_plan(int64_t n, int64_t n_rows)
{
    SortPlan p{};
    const int bits = key_bits(n_rows);
    p.bits = bits;
    p.npass = (bits + kMaxDigitBits - 1) / kMaxDigitBits;
    p.digit_bits = (bits + p.npass - 1) / p.npass;
    if (p.digit_bits < 2) p.digit_bits = 2;  // the scatter step reads histogram bins four at a time
    p.nblocks = n > 0 ? ceil_div(n, kKeysPerBlock) : 1;
    size_t o = 0;
    const size_t n4 = align_up(sizeof(uint32_t) * (size_t)(n > 0 ? n : 1));
    p.off_keys0 = o, o += n4;
    p.off_keys1 = o, o += n4;
    p.off_vals = o, o += n4;
    // per-block digit histograms: one table (multi-block sort) or one per pass (up to 65536 ids)
    const size_t hist_rows = n <= kMidMaxN ? (size_t)kMidMaxPass * mid_blocks(n) : (size_t)p.nblocks;
    p.off_hist = o, o += align_up(sizeof(uint32_t) * hist_rows * kMaxBins);
    p.off_totals = o, o += align_up(sizeof(uint32_t) * kMaxBins);
    p.off_heads = o, o += align_up(sizeof(uint32_t) * (size_t)p.nblocks);
    p.total = o;
    return p;
}

bool transr_grouped_path_ok(const kge_tables *tab, const kge_batch *bat);  // transr.hip

static int validate_job(const kge_inspect_job *job, Parts *parts, int64_t *n_out)
{
    if (job->n_parts < 1 || job->n_parts > 4) return KGE_EINVAL;
    if (job->n_rows <= 0 || job->n_rows > (int64_t(1) << 32)) return KGE_ESHAPE;
    parts->n_parts = job->n_parts;
    int64_t n = 0;
    for (int q = 0; q < job->n_parts; ++q) {
        if (job->part_len[q] < 0 || (job->part_len[q] > 0 && !job->parts[q])) return KGE_EINVAL;
        n += job->part_len[q];
        parts->p[q] = job->parts[q];
        parts->end[q] = n;
    }
    for (int q = job->n_parts; q < 4; ++q) parts->p[q] = job->parts[job->n_parts - 1], parts->end[q] = n;
    const kge_inspection *out = &job->out;
    if (n != out->n || n >= (int64_t(1) << 31)) return KGE_ESHAPE;
    if (!out->num_unique || !out->seg_offsets) return KGE_EINVAL;
    if (n > 0 && (!out->unique_ids || !out->perm || !out->inverse || !out->sorted_seg)) return KGE_EINVAL;
    if (!job->workspace || job->workspace_bytes < make_plan(n, job->n_rows).total) return KGE_EWORKSPACE;
    if (!aligned16(job->workspace)) return KGE_EWORKSPACE;  // the key buffers are read with 128-bit loads
    *n_out = n;
    return KGE_OK;
}

int plan_fused_inspection(const kge_inspect_job *jobs, int n_jobs, int slot, FusedInsp *out)
{
    if (!jobs || !out || slot < 0 || slot >= kFusedSlots || n_jobs < 1 || n_jobs > 2) return KGE_EINVAL;
    FusedInsp f{};
    f.n_jobs = n_jobs;
    int words = kMidDedupLdsWords;
    int blocks[2] = {0, 0};
    for (int q = 0; q < n_jobs; ++q) {
        Parts parts;
        int64_t n;
        const int rc = validate_job(&jobs[q], &parts, &n);
        if (rc) return rc;
        if (n < 1 || n > kMidMaxN) return KGE_EUNSUPPORTED;
        const int bits = key_bits(jobs[q].n_rows);
        if (bits > 2 * kMaxDigitBits) return KGE_EUNSUPPORTED;
        // two narrow digits rather than one wide one: the second pass hides inside its host kernel,
        // and the LDS a pass needs grows with the number of bins
        const SortPlan p = make_plan(n, jobs[q].n_rows);
        char *ws = static_cast<char *>(jobs[q].workspace);
        MidJob &J = f.j[q];
        J.parts = parts;
        J.n = n;
        J.npass = bits <= 6 ? 1 : 2;
        J.db = (bits + J.npass - 1) / J.npass;
        if (J.db < 2) J.db = 2;
        J.out = jobs[q].out;
        J.keys_final = reinterpret_cast<uint32_t *>(ws + p.off_keys0);
        J.keys_tmp = reinterpret_cast<uint32_t *>(ws + p.off_keys1);
        J.vals_tmp = reinterpret_cast<int32_t *>(ws + p.off_vals);
        J.hist = reinterpret_cast<uint32_t *>(ws + p.off_hist);
        blocks[q] = (int)ceil_div(n, kMidKeys);
        const int step = slot - (kFusedSlots - 2 - J.npass);
        const int w = step == 0 ? mid_hist_lds_words(1 << J.db, J.npass)
                                : (step >= 1 && step <= J.npass ? mid_pass_lds_words(1 << J.db, J.npass) : 0);
        words = w > words ? w : words;
    }
    f.split = blocks[0];
    f.blocks = (blocks[0] + blocks[1] + 7) / 8 * 8;
    f.slot = slot;
    f.lds_bytes = words * (int)sizeof(uint32_t);
    *out = f;
    return KGE_OK;
}

}  // namespace kge

using namespace kge;

extern "C" {

size_t kge_inspect_workspace(int64_t n, int64_t n_rows)
{
    if (n < 0 || n_rows <= 0) return 0;
    return make_plan(n, n_rows).total;
}

// multi-block path: 2-3 launches per digit pass + 2
static int inspect_large(const Parts &parts, int64_t n, int64_t n_rows, const kge_inspection *out, void *workspace,
                         hipStream_t st)
{
    const SortPlan p = make_plan(n, n_rows);
    char *ws = static_cast<char *>(workspace);
    uint32_t *keys_final = reinterpret_cast<uint32_t *>(ws + p.off_keys0);
    uint32_t *keys_tmp = reinterpret_cast<uint32_t *>(ws + p.off_keys1);
    int32_t *vals_tmp = reinterpret_cast<int32_t *>(ws + p.off_vals);
    uint32_t *hist = reinterpret_cast<uint32_t *>(ws + p.off_hist);
    uint32_t *totals = reinterpret_cast<uint32_t *>(ws + p.off_totals);
    uint32_t *heads = reinterpret_cast<uint32_t *>(ws + p.off_heads);
    const int nblocks = (int)p.nblocks;
    const int bins = 1 << p.digit_bits;
    if (n > 0) {
        const uint32_t *kin = nullptr;
        const int32_t *vin = nullptr;
        for (int pass = 0; pass < p.npass; ++pass) {
            const bool to_final = ((p.npass - 1 - pass) & 1) == 0;
            uint32_t *kout = to_final ? keys_final : keys_tmp;
            int32_t *vout = to_final ? out->perm : vals_tmp;
            const int shift = pass * p.digit_bits;
            const int fused = nblocks <= kFusedScanBlocks;
            hipLaunchKernelGGL(radix_hist_kernel, dim3(nblocks), dim3(kSortThreads), 0, st, parts, kin, n,
                               shift, bins, hist);
            if (!fused)
                hipLaunchKernelGGL(radix_colscan_kernel, dim3((bins + 255) / 256), dim3(256), 0, st, hist,
                                   totals, bins, nblocks);
            hipLaunchKernelGGL(radix_scatter_kernel, dim3(nblocks), dim3(kSortThreads), 0, st, parts, kin,
                               vin, n, shift, p.digit_bits, hist, totals, nblocks, fused, kout, vout);
            kin = kout;
            vin = vout;
        }
        hipLaunchKernelGGL(count_heads_kernel, dim3(nblocks), dim3(kSortThreads), 0, st, keys_final, n,
                           heads);
    }
    hipLaunchKernelGGL(finalize_kernel, dim3(nblocks), dim3(kSortThreads), 0, st, keys_final, out->perm, n,
                       heads, n > 0 ? nblocks : 0, *out);
    KGE_CHECK_LAUNCH();
    return KGE_OK;
}

int kge_inspect_batch(const kge_inspect_job *jobs, int n_jobs, void *stream)
{
    if (!jobs || n_jobs < 1 || n_jobs > 4) return KGE_EINVAL;
    hipStream_t st = as_stream(stream);
    Parts parts[4];
    int64_t n[4];
    for (int q = 0; q < n_jobs; ++q) {
        const int rc = validate_job(&jobs[q], &parts[q], &n[q]);
        if (rc) return rc;
    }
    MidJobs mid{};
    int n_mid = 0, max_pass = 0;
    int64_t mid_max = 0;
    for (int q = 0; q < n_jobs; ++q) {
        if (n[q] > kMidMaxN) {
            const int rc = inspect_large(parts[q], n[q], jobs[q].n_rows, &jobs[q].out, jobs[q].workspace, st);
            if (rc) return rc;
            continue;
        }
        const SortPlan p = make_plan(n[q], jobs[q].n_rows);
        char *ws = static_cast<char *>(jobs[q].workspace);
        MidJob &J = mid.j[n_mid++];
        J.parts = parts[q];
        J.n = n[q];
        J.npass = p.npass;
        J.db = p.digit_bits;
        J.out = jobs[q].out;
        J.keys_final = reinterpret_cast<uint32_t *>(ws + p.off_keys0);
        J.keys_tmp = reinterpret_cast<uint32_t *>(ws + p.off_keys1);
        J.vals_tmp = reinterpret_cast<int32_t *>(ws + p.off_vals);
        J.hist = reinterpret_cast<uint32_t *>(ws + p.off_hist);
        mid_max = n[q] > mid_max ? n[q] : mid_max;
        max_pass = p.npass > max_pass ? p.npass : max_pass;
    }
    if (n_mid > 0) {
        const dim3 grid((unsigned)(mid_max > 0 ? ceil_div(mid_max, kMidKeys) : 1), (unsigned)n_mid), block(kMidThreads);
        if (mid_max > 0) {
            hipLaunchKernelGGL(inspect_mid_hist_kernel, grid, block, 0, st, mid);
            for (int pass = 0; pass < max_pass; ++pass) {
                if (pass == 0) hipLaunchKernelGGL(inspect_mid_scatter_kernel<true>, grid, block, 0, st, mid, pass);
                else hipLaunchKernelGGL(inspect_mid_scatter_kernel<false>, grid, block, 0, st, mid, pass);
            }
        }
        // (jobs with a single digit pass are finished by their scatter step; empty jobs still need
        // the dedup step to write their zero counts)
        bool need_dedup = false;
        for (int q = 0; q < n_mid; ++q) need_dedup = need_dedup || mid.j[q].npass > 1 || mid.j[q].n == 0;
        if (need_dedup) hipLaunchKernelGGL(inspect_mid_dedup_kernel, grid, block, 0, st, mid);
        KGE_CHECK_LAUNCH();
    }
    return KGE_OK;
}

int kge_fused_inspection_ok(const kge_tables *tab, const kge_batch *bat, const kge_inspect_job *jobs)
{
    if (!tab || !bat || !jobs || bat->batch <= 0) return 0;
    switch (tab->model) {
    case KGE_TRANSE: case KGE_TRANSH: case KGE_DISTMULT: case KGE_COMPLEX: case KGE_ROTATE: case KGE_TRANSF:
        if (!bat->neg) return 0;  // the shared-negative kernels are the hosts
        break;
    case KGE_TRANSR: case KGE_RESCAL:
        if (bat->neg || !transr_grouped_path_ok(tab, bat)) return 0;  // the grouped MFMA kernels are the hosts
        break;
    default: return 0;
    }
    FusedInsp f;
    return plan_fused_inspection(jobs, fused_job_count(tab->model), 0, &f) == KGE_OK ? 1 : 0;
}

int kge_inspect(const int64_t *const *parts_in, const int64_t *part_len, int n_parts, int64_t n_rows,
                const kge_inspection *out, void *workspace, size_t workspace_bytes, void *stream)
{
    if (!out || !parts_in || !part_len || n_parts < 1 || n_parts > 4) return KGE_EINVAL;
    kge_inspect_job job{};
    for (int q = 0; q < n_parts; ++q) job.parts[q] = parts_in[q], job.part_len[q] = part_len[q];
    job.n_parts = n_parts;
    job.n_rows = n_rows;
    job.out = *out;
    job.workspace = workspace;
    job.workspace_bytes = workspace_bytes;
    return kge_inspect_batch(&job, 1, stream);
}

}  // extern "C"
