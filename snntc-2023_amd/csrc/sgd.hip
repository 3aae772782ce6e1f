// Plain SGD update of a network's weight tensors, w -= lr * dw, in ONE launch for all layers (the
// "SGD update" of a training step; the reference leaves it to the framework's optimizer,
// snntc/snntc-mnist.py:70).  A small network has a few weight tensors of very different sizes: one
// kernel per tensor pays a launch each, and a framework's multi-tensor kernel with its large
// per-block chunks fills only a few CUs.  Here every block owns SGD_BLOCK_ELEMS consecutive
// elements of one tensor; the (tensor, first block) table travels in the kernel arguments.
#include "snntc_common.h"

namespace snntc {
namespace {

constexpr int SGD_MAX_TENSORS = 32;
constexpr int SGD_THREADS = 256;
constexpr int SGD_BLOCK_ELEMS = SGD_THREADS * 4;      // one float4 per thread

struct SgdTable {
    float* w[SGD_MAX_TENSORS];
    const float* dw[SGD_MAX_TENSORS];
    long long n[SGD_MAX_TENSORS];
    int first_block[SGD_MAX_TENSORS + 1];             // prefix sums of the tensors' block counts
    int count;
};

__global__ void __launch_bounds__(SGD_THREADS) sgd_update_kernel(SgdTable tab, float lr) {
    const int block = blockIdx.x;
    int t = 0;
    while (t + 1 < tab.count && block >= tab.first_block[t + 1]) ++t;      // uniform, <= 31 steps
    float* __restrict__ w = tab.w[t];
    const float* __restrict__ dw = tab.dw[t];
    const long long n = tab.n[t];
    const long long e0 = ((long long)(block - tab.first_block[t]) * SGD_THREADS + threadIdx.x) * 4;
    if (e0 + 4 <= n && (((uintptr_t)w | (uintptr_t)dw) & 15) == 0) {
        float4 a = *reinterpret_cast<const float4*>(w + e0);
        const float4 g = *reinterpret_cast<const float4*>(dw + e0);
        a.x = __fmaf_rn(-lr, g.x, a.x);
        a.y = __fmaf_rn(-lr, g.y, a.y);
        a.z = __fmaf_rn(-lr, g.z, a.z);
        a.w = __fmaf_rn(-lr, g.w, a.w);
        *reinterpret_cast<float4*>(w + e0) = a;
    } else {
        for (long long e = e0; e < n && e < e0 + 4; ++e) w[e] = __fmaf_rn(-lr, dw[e], w[e]);
    }
}

}  // namespace

int launch_sgd_update(float* const* w, const float* const* dw, const int64_t* n, int count, float lr,
                      hipStream_t stream) {
    int t = 0;
    while (t < count) {
        SgdTable tab;
        tab.count = 0;
        int64_t blocks = 0;
        for (; t < count && tab.count < SGD_MAX_TENSORS; ++t) {
            if (n[t] <= 0) continue;
            tab.w[tab.count] = w[t];
            tab.dw[tab.count] = dw[t];
            tab.n[tab.count] = n[t];
            tab.first_block[tab.count] = (int)blocks;
            blocks += (n[t] + SGD_BLOCK_ELEMS - 1) / SGD_BLOCK_ELEMS;
            if (blocks > 0x7fffffffLL) return fail(SNNTC_ERR_TOO_LARGE, "sgd: grid too large");
            ++tab.count;
        }
        if (tab.count == 0) continue;
        tab.first_block[tab.count] = (int)blocks;
        {
            KernelTimerScope timer_("sgd_update", stream);
            hipLaunchKernelGGL(sgd_update_kernel, dim3((unsigned)blocks), dim3(SGD_THREADS), 0, stream, tab, lr);
        }
        SNNTC_HIP_CHECK(hipGetLastError());
    }
    return SNNTC_OK;
}

}  // namespace snntc
