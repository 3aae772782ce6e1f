// Earliest-spike pooling of NHWC spike times (SNN_maxpool2d, SNN_TC_Modules.py:215-246).
//
// The reference pads the input with padvalue (1e5, "never fired"), negates it, runs the
// framework's VALID max pooling and negates the result; its gradient follows the framework's
// argmax.  Here the padding is implicit (positions outside the image count as padvalue), the
// minimum is taken directly, and the forward pass records which window position attained it --
// the first one in (kh, kw) order, as a max pooling that replaces its running maximum only on a
// strictly greater value does -- so the backward pass is a gather: every input pixel adds the
// gradients of the windows that recorded it, in (kh, kw) order, with no atomics.
#include "snntc_common.h"

namespace snntc {
namespace {

// Division of a small non-negative number by a launch constant without the divide sequence:
// n / d == umulhi(n, 2^32 / d + 1) as long as n * d < 2^32.  The host leaves `magic` at 0 where that
// bound does not hold (and for d == 1), which selects the plain division.
struct FastDiv {
    unsigned d, magic;
};
__device__ __forceinline__ unsigned fast_div(unsigned n, FastDiv f) {
    return f.magic ? __umulhi(n, f.magic) : (f.d == 1 ? n : n / f.d);
}
FastDiv make_fast_div(int64_t d, int64_t max_n) {
    FastDiv f{(unsigned)d, 0u};
    if (d > 1 && max_n * d < (int64_t)1 << 32) f.magic = (unsigned)(0xffffffffu / (unsigned)d + 1u);
    return f;
}

// blockIdx.x = output row (b, nh), blockIdx.y * 256 + threadIdx.x = (nw, c) within the row: 32-bit index
// arithmetic only, consecutive lanes on consecutive channels.
__global__ void __launch_bounds__(256)
min_pool_forward_kernel(const float* __restrict__ x, float* __restrict__ y, int32_t* __restrict__ arg, int H, int W,
                        int C, int Kh, int Kw, int Sh, int Sw, int pad_top, int pad_left, int Nh, int Nw,
                        float pad_value, FastDiv by_c) {
    const unsigned e = blockIdx.y * 256u + threadIdx.x;
    if (e >= (unsigned)(Nw * C)) return;
    const unsigned nw = fast_div(e, by_c), c = e - nw * (unsigned)C;
    const unsigned row = blockIdx.x;
    const unsigned b = row / (unsigned)Nh, nh = row - b * (unsigned)Nh;                    // scalar: once per block
    const int h0 = (int)nh * Sh - pad_top, w0 = (int)nw * Sw - pad_left;
    const float* __restrict__ img = x + (size_t)b * H * W * C + c;
    float best = INFINITY;
    int where = 0;
    for (int kh = 0; kh < Kh; ++kh) {
        const int h = h0 + kh;
        for (int kw = 0; kw < Kw; ++kw) {
            const int w = w0 + kw;
            const float v = (h >= 0 && h < H && w >= 0 && w < W) ? img[((size_t)h * W + w) * C] : pad_value;
            if (v < best) { best = v; where = kh * Kw + kw; }
        }
    }
    const size_t t = (size_t)row * Nw * C + e;
    y[t] = best;
    if (arg) arg[t] = where;
}

// blockIdx.x = input row (b, h), blockIdx.y * 256 + threadIdx.x = (w, c) within the row.
__global__ void __launch_bounds__(256)
min_pool_backward_kernel(const float* __restrict__ gy, const int32_t* __restrict__ arg, float* __restrict__ dx,
                         int H, int W, int C, int Kh, int Kw, int Sh, int Sw, int pad_top, int pad_left, int Nh,
                         int Nw, FastDiv by_c, FastDiv by_sw) {
    const unsigned e = blockIdx.y * 256u + threadIdx.x;
    if (e >= (unsigned)(W * C)) return;
    const int w = (int)fast_div(e, by_c), c = (int)e - w * C;
    const unsigned row = blockIdx.x;
    const unsigned b = row / (unsigned)H;
    const int h = (int)(row - b * (unsigned)H);
    // the windows that cover the pixel: nh*Sh - pad_top <= h < nh*Sh - pad_top + Kh, likewise nw;
    // walking them from the last to the first visits the window positions in (kh, kw) order
    const int hp = h + pad_top, wp = w + pad_left;
    const int nh_hi = min(Nh - 1, hp / Sh), nh_lo = hp - Kh + 1 <= 0 ? 0 : (hp - Kh + Sh) / Sh;   // scalar
    const int nw_hi = min(Nw - 1, (int)fast_div((unsigned)wp, by_sw));
    const int nw_lo = wp - Kw + 1 <= 0 ? 0 : (int)fast_div((unsigned)(wp - Kw + Sw), by_sw);
    float sum = 0.0f;
    for (int nh = nh_hi; nh >= nh_lo; --nh) {
        const int kh = hp - nh * Sh;
        for (int nw = nw_hi; nw >= nw_lo; --nw) {
            const int kw = wp - nw * Sw;
            const size_t o = (((size_t)b * Nh + nh) * Nw + nw) * C + c;
            if (arg[o] == kh * Kw + kw) sum += gy[o];
        }
    }
    dx[(size_t)row * W * C + e] = sum;
}

}  // namespace

int launch_min_pool_forward(const float* x, float* y, int32_t* arg, const PoolGeom& g, float pad_value,
                            hipStream_t stream) {
    const int64_t rows = g.B * g.Nh, per_row = g.Nw * g.C;
    if (rows <= 0 || per_row <= 0) return SNNTC_OK;
    dim3 grid((unsigned)rows, (unsigned)((per_row + 255) / 256));
    if (grid.y > 65535u) return fail(SNNTC_ERR_TOO_LARGE, "pooling: output row of %lld elements too long", (long long)per_row);
    {
        KernelTimerScope timer_("min_pool", stream);
        hipLaunchKernelGGL(min_pool_forward_kernel, grid, dim3(256), 0, stream, x, y, arg, (int)g.H, (int)g.W, (int)g.C,
                           (int)g.Kh, (int)g.Kw, (int)g.Sh, (int)g.Sw, (int)g.pad_top, (int)g.pad_left, (int)g.Nh,
                           (int)g.Nw, pad_value, make_fast_div(g.C, per_row));
    }
    SNNTC_HIP_CHECK(hipGetLastError());
    return SNNTC_OK;
}

int launch_min_pool_backward(const float* gy, const int32_t* arg, float* dx, const PoolGeom& g, hipStream_t stream) {
    const int64_t rows = g.B * g.H, per_row = g.W * g.C;
    if (rows <= 0 || per_row <= 0) return SNNTC_OK;
    dim3 grid((unsigned)rows, (unsigned)((per_row + 255) / 256));
    if (grid.y > 65535u) return fail(SNNTC_ERR_TOO_LARGE, "pooling: input row of %lld elements too long", (long long)per_row);
    {
        KernelTimerScope timer_("min_pool_grad", stream);
        hipLaunchKernelGGL(min_pool_backward_kernel, grid, dim3(256), 0, stream, gy, arg, dx, (int)g.H, (int)g.W,
                           (int)g.C, (int)g.Kh, (int)g.Kw, (int)g.Sh, (int)g.Sw, (int)g.pad_top, (int)g.pad_left,
                           (int)g.Nh, (int)g.Nw, make_fast_div(g.C, per_row), make_fast_div(g.Sw, g.W + g.Kw + g.Sw));
    }
    SNNTC_HIP_CHECK(hipGetLastError());
    return SNNTC_OK;
}

}  // namespace snntc
