// Atomic-free segmented reduction: the backward pass produces one gradient row per OCCURRENCE
// of a table row; the inspection's stable sort puts the occurrences of one id next to each
// other, and each output row is the sum of its run, written exactly once.
//
// Level 1: a wave owns kSegL consecutive sorted positions (and one 256-float column chunk of
// the rows).  All its row loads are issued at once; then the positions are walked in order.
// A run that lies wholly inside the block is final.  A run that began in an earlier block is
// stored to partial slot 0 of the block, one that continues past the block to slot 1.
// Level 2: the block in which a long run STARTS adds that run's slot-1 partial and the slot-0
// partials of the following blocks (four waves share the blocks, combined through LDS).
// The summation order is fixed by the sorted order, so results are deterministic.
#include "seg_reduce.hpp"

namespace kge {

// The rider's sums: a work item is (sum i, 256 float4 of the row); the slice's workgroups stride over the items.
__device__ __forceinline__ void sum_rider_body(const SumRider &r)
{
    const int nsum = r.num[0] < r.max_sums ? r.num[0] : r.max_sums;
    const int64_t q4 = r.row_floats / 4;
    const int64_t nb = (q4 + 255) / 256;
    for (int64_t it = blockIdx.x; it < nsum * nb; it += gridDim.x) {
        const int i = (int)(it / nb);
        const int64_t f = (it % nb) * 256 + threadIdx.x;
        if (f >= q4) continue;
        const int cnt = r.cnt[i];
        const float4 *src = reinterpret_cast<const float4 *>(r.part) + (int64_t)r.first[i] * q4 + f;
        float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
        constexpr int kFly = 8;  // rows in flight: unconditional loads (a row past the end re-reads the last one), masked afterwards
        for (int c0 = 0; c0 < cnt; c0 += kFly) {
            float4 v[kFly];
#pragma unroll
            for (int u = 0; u < kFly; ++u) v[u] = src[(int64_t)(c0 + u < cnt ? c0 + u : cnt - 1) * q4];
#pragma unroll
            for (int u = 0; u < kFly; ++u)
                if (c0 + u < cnt) acc.x += v[u].x, acc.y += v[u].y, acc.z += v[u].z, acc.w += v[u].w;
        }
        reinterpret_cast<float4 *>(r.out)[(int64_t)r.seg[i] * q4 + f] = acc;
    }
}

template <int V>
__global__ __launch_bounds__(256) void seg_reduce_l1(SegArgs3 jobs, SumRider rider)
{
    if (rider.max_sums > 0 && blockIdx.y == gridDim.y - 1) {  // the last slice of the grid is the rider's
        sum_rider_body(rider);
        return;
    }
    seg_l1_wave<V>(jobs.j[blockIdx.y], (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6));
}

// One workgroup per (block, chunk of 64 V columns): the column chunks of a wide row are independent
// chains of round trips and run side by side (nch = chunks of the widest job of the launch).
template <int V>
__global__ __launch_bounds__(256) void seg_reduce_l2(SegArgs3 jobs, int nch, SumRider rider)
{
    __shared__ float s_part[4][kWave * 4];
    if (rider.max_sums > 0 && blockIdx.y == gridDim.y - 1) {  // (when level 1 rode in the launch the sums depend on)
        sum_rider_body(rider);
        return;
    }
    const SegArgs &a = jobs.j[blockIdx.y];
    const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x >> 6;
    const int64_t j = blockIdx.x / nch;
    const int c0 = (int)(blockIdx.x % nch) * kWave * V;
    const int64_t p0 = j * kSegL;
    if (p0 >= a.n || c0 >= a.d) return;  // uniform for the workgroup
    const int64_t p1 = p0 + kSegL < a.n ? p0 + kSegL : a.n;
    const int sg = a.sorted_seg[p1 - 1];
    const int s0 = a.seg_offsets[sg], s1 = a.seg_offsets[sg + 1];
    if (s1 <= p0 + kSegL || s0 < p0) return;  // no run starts here and continues
    const int64_t je = (s1 - 1) / kSegL;
    const int d = a.d;
    {
        const int colv = c0 + lane * V;
        const bool active = colv < d;
        Vec<V> acc;
#pragma unroll
        for (int e = 0; e < V; ++e) acc.v[e] = 0.0f;
        constexpr int kFly = 8;  // partial rows in flight per wave: the hottest row's chain is the long pole
        for (int64_t jj = j + 1 + wave; jj <= je; jj += 4 * kFly) {
            Vec<V> t[kFly];
#pragma unroll
            for (int u = 0; u < kFly; ++u) {
                const int64_t jb = jj + 4 * u;
                t[u] = Vec<V>::load(a.partial + ((jb <= je ? jb : je) * 2) * (int64_t)d + (active ? colv : 0));
            }
#pragma unroll
            for (int u = 0; u < kFly; ++u)
                if (jj + 4 * u > je) {
#pragma unroll
                    for (int e = 0; e < V; ++e) t[u].v[e] = 0.0f;
                }
#pragma unroll
            for (int u = 0; u < kFly; ++u)
#pragma unroll
                for (int e = 0; e < V; ++e) acc.v[e] += t[u].v[e];
        }
#pragma unroll
        for (int e = 0; e < V; ++e) s_part[wave][lane * V + e] = acc.v[e];
        __syncthreads();
        if (wave == 0 && active) {
            Vec<V> r = Vec<V>::load(a.partial + (j * 2 + 1) * (int64_t)d + colv);
#pragma unroll
            for (int e = 0; e < V; ++e)
                r.v[e] += (s_part[0][lane * V + e] + s_part[1][lane * V + e]) +
                          (s_part[2][lane * V + e] + s_part[3][lane * V + e]);
            r.store(a.out + (int64_t)sg * d + colv);
        }
    }
}

// Kernel arguments and grid of the level-1 pass over `jobs`.
static int plan_jobs(const SegJob *jobs, int n_jobs, SegL1Rider *out, int64_t *max_blocks, int64_t *max_nch)
{
    SegL1Rider r{};
    int m = 0;
    int64_t max_waves = 0;
    *max_blocks = 0, *max_nch = 1;
    bool v4 = true;
    for (int q = 0; q < n_jobs && m < 3; ++q) {
        const SegJob &jb = jobs[q];
        if (!jb.ins || jb.ins->n == 0 || jb.d == 0) continue;
        r.jobs.j[m] = SegArgs{jb.occ, jb.identity_perm ? nullptr : jb.ins->perm, jb.ins->sorted_seg,
                              jb.ins->seg_offsets, jb.ins->n, jb.d, jb.out, jb.partial,
                              jb.scale_num, jb.scale_den, (jb.scaled ? 1 : 0) | (jb.sign_rows ? 2 : 0), (int)jb.wrap};
        v4 = v4 && jb.d % 4 == 0 && aligned16(jb.occ) && aligned16(jb.out) && aligned16(jb.partial);
        ++m;
    }
    for (int q = 0; q < m; ++q) {
        const int V = v4 ? 4 : 1;
        const int64_t nblk = ceil_div(r.jobs.j[q].n, kSegL);
        const int64_t nch = ceil_div(r.jobs.j[q].d, kWave * V);
        max_waves = nblk * nch > max_waves ? nblk * nch : max_waves;
        *max_blocks = nblk > *max_blocks ? nblk : *max_blocks;
        *max_nch = nch > *max_nch ? nch : *max_nch;
    }
    for (int q = m; q < 3; ++q) r.jobs.j[q] = r.jobs.j[0], r.jobs.j[q].n = 0;  // unused slots do nothing
    r.n_jobs = m, r.v4 = v4 ? 1 : 0;
    r.blocks_x = (int)ceil_div(max_waves, 4);
    *out = r;
    return m;
}

SegL1Rider plan_seg_l1_rider(const SegJob *jobs, int n_jobs)
{
    SegL1Rider r{};
    int64_t mb, mn;
    plan_jobs(jobs, n_jobs, &r, &mb, &mn);
    return r;
}

int launch_seg_reduce_jobs(const SegJob *jobs, int n_jobs, hipStream_t st, kge_timeline *timeline, const SumRider *rider,
                           bool level1_rode)
{
    const SumRider rd = rider && rider->max_sums > 0 ? *rider : SumRider{};
    if (rd.max_sums > 0 && (rd.row_floats % 4 != 0 || !aligned16(rd.part) || !aligned16(rd.out))) return KGE_EINVAL;
    SegL1Rider pl{};
    int64_t max_blocks = 0, max_nch = 1;
    const int m = plan_jobs(jobs, n_jobs, &pl, &max_blocks, &max_nch);
    if (m == 0 && rd.max_sums == 0) return KGE_OK;
    const SegArgs3 &args = pl.jobs;
    const bool v4 = pl.v4 != 0;
    const SumRider none{};
    int64_t g1x = pl.blocks_x;
    if (rd.max_sums > 0 && g1x < 256) g1x = 256;  // (a small reduction still gives the rider a grid's worth of workgroups)
    int64_t g2x = max_blocks * max_nch;
    if (level1_rode && rd.max_sums > 0 && g2x < 256) g2x = 256;
    const bool r1 = !level1_rode && rd.max_sums > 0, r2 = level1_rode && rd.max_sums > 0;
    const dim3 g1((unsigned)g1x, (unsigned)(m + (r1 ? 1 : 0))), g2((unsigned)g2x, (unsigned)(m + (r2 ? 1 : 0))), block(256);
    const bool level2 = m > 0 || r2;
    if (v4) {
        if (!level1_rode) {
            hipLaunchKernelGGL(seg_reduce_l1<4>, g1, block, 0, st, args, r1 ? rd : none);
            timeline_mark(timeline, st, "seg_reduce_l1");
        }
        if (level2) hipLaunchKernelGGL(seg_reduce_l2<4>, g2, block, 0, st, args, (int)max_nch, r2 ? rd : none);
    } else {
        if (!level1_rode) {
            hipLaunchKernelGGL(seg_reduce_l1<1>, g1, block, 0, st, args, r1 ? rd : none);
            timeline_mark(timeline, st, "seg_reduce_l1");
        }
        if (level2) hipLaunchKernelGGL(seg_reduce_l2<1>, g2, block, 0, st, args, (int)max_nch, r2 ? rd : none);
    }
    if (level2) timeline_mark(timeline, st, "seg_reduce_l2");
    KGE_CHECK_LAUNCH();
    return KGE_OK;
}

}  // namespace kge
