// Loss of the reference's example networks: mean categorical cross-entropy of a one-hot label
// against softmax(-t), t = output spike times (SNN_TC_Modules.py:286-288) -- the earliest output
// spike is the predicted class.  One kernel produces the per-sample loss and the gradient of the
// batch mean with respect to the spike times; as separate framework ops this is a dozen launches
// of a few microseconds each, a visible share of a small network's training step.
#include "snntc_common.h"

namespace snntc {
namespace {

__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int d = kWave / 2; d > 0; d >>= 1) v = fmaxf(v, __shfl_xor(v, d, kWave));
    return v;
}
__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int d = kWave / 2; d > 0; d >>= 1) v += __shfl_xor(v, d, kWave);
    return v;
}

// One wavefront per sample.  With l = -t, p = softmax(l), T = sum_j label_j:
//   loss_b = -sum_j label_j * (l_j - logsumexp(l)),   d(mean loss)/dt_j = (label_j - p_j * T) / B
__global__ void __launch_bounds__(256)
softmax_time_loss_kernel(const float* __restrict__ times, const float* __restrict__ label,
                         float* __restrict__ sample_loss, float* __restrict__ dtimes, int B, int J, float inv_b) {
    const int lane = threadIdx.x % kWave;
    const int b = blockIdx.x * (blockDim.x / kWave) + threadIdx.x / kWave;
    if (b >= B) return;
    const float* __restrict__ t = times + (size_t)b * J;
    const float* __restrict__ y = label + (size_t)b * J;
    float m = -INFINITY;
    for (int j = lane; j < J; j += kWave) m = fmaxf(m, -t[j]);
    m = wave_max(m);
    float se = 0.0f, dot = 0.0f, tot = 0.0f;
    for (int j = lane; j < J; j += kWave) {
        const float l = -t[j] - m;
        se += expf(l);
        dot += y[j] * l;
        tot += y[j];
    }
    se = wave_sum(se); dot = wave_sum(dot); tot = wave_sum(tot);
    const float lse = logf(se);
    if (lane == 0 && sample_loss) sample_loss[b] = tot * lse - dot;      // -sum_j y_j (l_j - lse)
    if (dtimes) {
        float* __restrict__ g = dtimes + (size_t)b * J;
        const float scale = tot / se;
        for (int j = lane; j < J; j += kWave) g[j] = (y[j] - expf(-t[j] - m) * scale) * inv_b;
    }
}

}  // namespace

int launch_softmax_time_loss(const float* times, const float* label, float* sample_loss, float* dtimes,
                             int64_t B, int64_t J, hipStream_t stream) {
    if (B <= 0 || J <= 0) return SNNTC_OK;
    const int waves_per_block = 4;
    const int64_t blocks = (B + waves_per_block - 1) / waves_per_block;
    if (blocks > 0x7fffffffLL) return fail(SNNTC_ERR_TOO_LARGE, "loss: too many samples");
    {
        KernelTimerScope timer_("softmax_time_loss", stream);
        hipLaunchKernelGGL(softmax_time_loss_kernel, dim3((unsigned)blocks), dim3(256), 0, stream, times, label,
                           sample_loss, dtimes, (int)B, (int)J, 1.0f / (float)B);
    }
    SNNTC_HIP_CHECK(hipGetLastError());
    return SNNTC_OK;
}

}  // namespace snntc
