// Causal-set scan: for every (segment, output neuron) walk the segment's inputs in ascending
// order, accumulate sum(w) and sum(w*z), and stop at the first prefix whose weighted mean lies
// after its last input and not after the next one.
//
// Replaces SnnFcCudaOutKernel / SnnFcCudaOutKernelBias (snntc/snnfc_kernels.cu.cc:19-71,
// snntc/snncv_kernels.cu.cc:19-72) and reproduces their arithmetic step by step: bias first,
// sequential fp32 accumulation with a fused multiply-add for ysum, the division-free firing test
// |ysum| > x*|wsum| with the product rounded on its own, and y = ysum * (1/wsum).
//
// Mapping: one wavefront per (segment, block of 64 neurons); lanes run across neurons, so the
// weight row w[perm[k], j0..j0+63] is one coalesced 256-byte read and the sorted value / index
// of step k are the same for every lane (fetched through the scalar path).  Steps are taken in
// chunks of CHUNK so the weight reads of a chunk are in flight together; lanes that have closed
// their causal set idle until the whole wavefront has, then the wavefront leaves the loop.
#include "snntc_common.h"

namespace snntc {
namespace {

constexpr int CHUNK = 8;

template <bool WANT_K>
__global__ void __launch_bounds__(256)
scan_kernel(const float* __restrict__ sorted, const int32_t* __restrict__ perm,
            const float* __restrict__ w, float* __restrict__ y_out, float* __restrict__ rcp_out,
            int32_t* __restrict__ k_out, int64_t n_items, int S, int I, int J, int j_blocks,
            NeuronParams np) {
    // work item = (segment, 64-neuron block); one per wavefront
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
    const int64_t item = (int64_t)blockIdx.x * (blockDim.x / kWave) + wave;
    if (item >= n_items) return;
    const int seg = (int)(item / j_blocks);
    const int jb = (int)(item - (int64_t)seg * j_blocks);
    const int lane = threadIdx.x % kWave;
    const int j = jb * kWave + lane;
    const bool active = j < J;
    const int jc = active ? j : J - 1;          // clamp so every lane reads valid memory

    const float* __restrict__ xs = sorted + (size_t)seg * I;
    const int32_t* __restrict__ pr = perm + (size_t)seg * I;
    const float* __restrict__ wcol = w + jc;

    // number of real inputs: first sorted position whose value exceeds MAX-0.1 (binary search)
    int n = 0;
    {
        int lo = 0, hi = I;
        while (lo < hi) {
            const int mid = (lo + hi) >> 1;
            if (xs[mid] > np.max_cmp) hi = mid; else lo = mid + 1;
        }
        n = lo;
    }

    float wsum = -np.theta, ysum = 0.0f, wa = 0.0f, ya = 0.0f;
    bool fired = false;
    if (np.bias) {
        const float wb = wcol[(size_t)I * J];
        wsum += wb;
        ysum = np.biasvolt * wb;
        wa = fabsf(wsum);
        ya = wsum < 0.0f ? -ysum : ysum;
        fired = ya > wa * np.biasvolt;
    }

    bool done = !active;
    int kcnt = 0;
    for (int k0 = 0; k0 < n; k0 += CHUNK) {
        float xv[CHUNK], wv[CHUNK];
#pragma unroll
        for (int u = 0; u < CHUNK; ++u) {
            const int kk = min(k0 + u, n - 1);
            xv[u] = xs[kk];
            wv[u] = wcol[(size_t)pr[kk] * J];
        }
#pragma unroll
        for (int u = 0; u < CHUNK; ++u) {
            if (k0 + u < n && !done) {
                const float x = xv[u];
                if (fired && ya <= x * wa) {
                    done = true;
                } else {
                    wsum += wv[u];
                    ysum = __fmaf_rn(x, wv[u], ysum);
                    wa = fabsf(wsum);
                    ya = wsum < 0.0f ? -ysum : ysum;
                    fired = ya > x * wa;
                    if (WANT_K) kcnt = k0 + u + 1;
                }
            }
        }
        if (__all(done)) break;
    }

    if (active) {
        float y = np.max_time, r = 0.0f;
        if (fired) {
            r = 1.0f / wsum;
            y = ysum * r;
            if (y >= np.max_time) { y = np.max_time; r = 0.0f; }
        }
        const size_t o = (size_t)seg * J + j;
        y_out[o] = y;
        rcp_out[o] = r;
        if (WANT_K) k_out[o] = (fired && r != 0.0f) ? kcnt : -1;
    }
}

}  // namespace

int launch_scan(const float* sorted, const int32_t* perm, const float* w, float* y, float* rcp,
                int32_t* causal_k, int64_t S, int64_t I, int64_t J, const NeuronParams& np,
                hipStream_t stream) {
    if (S <= 0 || J <= 0) return SNNTC_OK;
    const int j_blocks = (int)((J + kWave - 1) / kWave);
    const int64_t n_items = S * j_blocks;
    const int waves_per_block = 4;
    const int64_t blocks = (n_items + waves_per_block - 1) / waves_per_block;
    if (blocks > 0x7fffffffLL) return fail(SNNTC_ERR_TOO_LARGE, "scan: grid too large");
    dim3 grid((unsigned)blocks), block(waves_per_block * kWave);
    {
        KernelTimerScope timer_("scan", stream);
        if (causal_k)
            hipLaunchKernelGGL(scan_kernel<true>, grid, block, 0, stream, sorted, perm, w, y, rcp, causal_k,
                               n_items, (int)S, (int)I, (int)J, j_blocks, np);
        else
            hipLaunchKernelGGL(scan_kernel<false>, grid, block, 0, stream, sorted, perm, w, y, rcp, causal_k,
                               n_items, (int)S, (int)I, (int)J, j_blocks, np);
    }
    SNNTC_HIP_CHECK(hipGetLastError());
    return SNNTC_OK;
}

}  // namespace snntc
