// Margin-ranking loss over (positive, shared-negative) score pairs and its gradient.
// Not part of the reference (it has no loss); defined as
//   L = mean_{b,k} max(0, margin - sign * (pos[b] - neg[b][k])).
#include <mutex>

#include "common.hpp"

namespace kge {

constexpr int kLossWaves = 4;

__global__ __launch_bounds__(kLossWaves *kWave) void margin_rows_kernel(
    const float *pos, const float *neg, int64_t B, int64_t N, float margin, float sign, float inv,
    float *dpos, float *dneg, double *row_loss)
{
    const int lane = threadIdx.x & (kWave - 1);
    const int64_t b = (int64_t)blockIdx.x * kLossWaves + (threadIdx.x >> 6);
    if (b >= B) return;
    const float p = pos[b];
    float sum = 0.0f;
    int cnt = 0;
    for (int64_t k = lane; k < N; k += kWave) {
        const float v = margin - sign * (p - neg[b * N + k]);
        const bool on = v > 0.0f;
        sum += on ? v : 0.0f;
        cnt += on ? 1 : 0;
        if (dneg) dneg[b * N + k] = on ? sign * inv : 0.0f;
    }
    sum = wave_sum(sum);
    cnt = wave_sum_i(cnt);
    if (lane == 0) {
        row_loss[b] = (double)sum;
        if (dpos) dpos[b] = -sign * inv * (float)cnt;
    }
}

__global__ __launch_bounds__(256) void margin_total_kernel(const double *row_loss, int64_t B, double scale,
                                                           float *loss)
{
    __shared__ double s[256];
    double acc = 0.0;
    for (int64_t i = threadIdx.x; i < B; i += 256) acc += row_loss[i];
    s[threadIdx.x] = acc;
    __syncthreads();
    for (int o = 128; o > 0; o >>= 1) {
        if ((int)threadIdx.x < o) s[threadIdx.x] += s[threadIdx.x + o];
        __syncthreads();
    }
    if (threadIdx.x == 0) loss[0] = (float)(s[0] * scale);
}

// Scratch of kge_margin_loss_static: the per-row partial losses, one double per positive.  Every
// GPU the library runs on holds its own copy of this array (512 KiB) until the process ends.
constexpr int64_t kStaticLossRows = KGE_MARGIN_LOSS_STATIC_MAX_BATCH;
static __device__ __align__(256) double scratch[kStaticLossRows];

constexpr int kMaxDevices = 64;
static std::mutex g_scratch_mutex;
static double *g_scratch_ptr[kMaxDevices];  // device address of `scratch` on each device, once looked up

// Device address of `scratch` on the current device (the array's name is only a host-side handle).
static int static_scratch(double **out)
{
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return KGE_ELAUNCH;
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (!g_scratch_ptr[dev]) {
        void *p = nullptr;
        if (hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)) != hipSuccess || !p) return KGE_ELAUNCH;
        g_scratch_ptr[dev] = static_cast<double *>(p);
    }
    *out = g_scratch_ptr[dev];
    return KGE_OK;
}

}  // namespace kge

using namespace kge;

extern "C" {

size_t kge_margin_loss_workspace(int64_t batch, int64_t n_neg)
{
    (void)n_neg;
    return batch > 0 ? sizeof(double) * (size_t)batch : 0;
}

int kge_margin_loss(const float *pos, const float *neg, int64_t batch, int64_t n_neg, float margin,
                    float sign, float *loss, float *dpos, float *dneg, void *workspace,
                    size_t workspace_bytes, void *stream)
{
    if (batch < 0 || n_neg < 0 || !loss) return KGE_EINVAL;
    if (batch > 0 && n_neg > 0 && (!pos || !neg)) return KGE_EINVAL;
    if (batch > 0 && (!workspace || workspace_bytes < sizeof(double) * (size_t)batch)) return KGE_EWORKSPACE;
    hipStream_t st = as_stream(stream);
    const double count = (double)batch * (double)n_neg;
    const float inv = count > 0 ? (float)(1.0 / count) : 0.0f;
    double *rows = static_cast<double *>(workspace);
    if (batch > 0)
        hipLaunchKernelGGL(margin_rows_kernel, dim3((unsigned)ceil_div(batch, kLossWaves)),
                           dim3(kLossWaves * kWave), 0, st, pos, neg, batch, n_neg, margin, sign, inv, dpos,
                           dneg, rows);
    hipLaunchKernelGGL(margin_total_kernel, dim3(1), dim3(256), 0, st, rows, batch,
                       count > 0 ? 1.0 / count : 0.0, loss);
    KGE_CHECK_LAUNCH();
    return KGE_OK;
}

int kge_margin_loss_static(const float *pos, const float *neg, int64_t batch, int64_t n_neg, float margin,
                           float sign, float *loss, float *dpos, float *dneg, void *stream)
{
    if (batch > kStaticLossRows) return KGE_EWORKSPACE;  // more rows than the built-in scratch holds
    double *rows = nullptr;
    const int rc = static_scratch(&rows);
    if (rc) return rc;
    // every row slot the total kernel reads is written by the row kernel of the same call first,
    // so nothing left behind by an earlier call needs clearing
    return kge_margin_loss(pos, neg, batch, n_neg, margin, sign, loss, dpos, dneg, rows,
                           sizeof(double) * (size_t)kStaticLossRows, stream);
}

}  // extern "C"
