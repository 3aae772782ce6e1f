// Earliest-spike pooling of NHWC spike times (SNN_maxpool2d, SNN_TC_Modules.py:215-246).
//
// The reference pads the input with padvalue (1e5, "never fired"), negates it, runs the
// framework's VALID max pooling and negates the result; its gradient follows the framework's
// argmax.  Here the padding is implicit (positions outside the image count as padvalue), the
// minimum is taken directly, and the forward pass records which window position attained it --
// the first one in (kh, kw) order, as a max pooling that replaces its running maximum only on a
// strictly greater value does -- so the backward pass is a gather: every input pixel adds the
// gradients of the windows that recorded it, in (kh, kw) order, with no atomics.
//
// Also here: the SAME padding of SNN_conv (SNN_TC_Modules.py:147-161, tf.pad with MAX_SPIKE_TIME) as
// one pass that writes every element of the padded tensor once, and the matching crop of the gradient.
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

// blockIdx.x = output row (b, nh); a thread takes VEC consecutive channels of one (nw, c) position of
// the row (VEC = 4 when C is a multiple of 4 and the tensors are 16-byte aligned): 32-bit index
// arithmetic only, consecutive lanes on consecutive channels.
template <int VEC>
__global__ void __launch_bounds__(256)
min_pool_forward_kernel(const float* __restrict__ x, float* __restrict__ y, int32_t* __restrict__ arg, int H, int W,
                        int C, int Kh, int Kw, int Sh, int Sw, int pad_top, int pad_left, int Nh, int Nw,
                        float pad_value, FastDiv by_c, TimeCopy copy) {
    const unsigned e = (blockIdx.y * 256u + threadIdx.x) * VEC;
    if (e >= (unsigned)(Nw * C)) return;
    const unsigned nw = fast_div(e, by_c), c = e - nw * (unsigned)C;
    const unsigned row = blockIdx.x;
    const unsigned b = row / (unsigned)Nh, nh = row - b * (unsigned)Nh;                    // scalar: once per block
    const int h0 = (int)nh * Sh - pad_top, w0 = (int)nw * Sw - pad_left;
    const float* __restrict__ img = x + (size_t)b * H * W * C + c;
    float best[VEC];
    int where[VEC];
#pragma unroll
    for (int v = 0; v < VEC; ++v) { best[v] = INFINITY; where[v] = 0; }
    for (int kh = 0; kh < Kh; ++kh) {
        const int h = h0 + kh;
        for (int kw = 0; kw < Kw; ++kw) {
            const int w = w0 + kw;
            float val[VEC];
#pragma unroll
            for (int v = 0; v < VEC; ++v) val[v] = pad_value;
            if (h >= 0 && h < H && w >= 0 && w < W) {
                const float* p = img + ((size_t)h * W + w) * C;
                if (VEC == 4) {
                    const float4 q = *reinterpret_cast<const float4*>(p);
                    val[0] = q.x; val[1] = q.y; val[2] = q.z; val[3] = q.w;
                } else {
                    val[0] = *p;
                }
            }
#pragma unroll
            for (int v = 0; v < VEC; ++v)
                if (val[v] < best[v]) { best[v] = val[v]; where[v] = kh * Kw + kw; }
        }
    }
    const size_t t = (size_t)row * Nw * C + e;
    if (VEC == 4) {
        *reinterpret_cast<float4*>(y + t) = make_float4(best[0], best[1], best[2], best[3]);
        if (arg) *reinterpret_cast<int4*>(arg + t) = make_int4(where[0], where[1], where[2], where[3]);
    } else {
        y[t] = best[0];
        if (arg) arg[t] = where[0];
    }
    if (copy.dst) {                                      // the same times inside the next layer's padded input
        float* q = copy.dst + (((size_t)b * copy.h + nh + copy.top) * copy.w + nw + copy.left) * C + c;
        if (VEC == 4) *reinterpret_cast<float4*>(q) = make_float4(best[0], best[1], best[2], best[3]);
        else *q = best[0];
    }
}

// blockIdx.x = input row (b, h); a thread takes VEC consecutive channels of one (w, c) position.
template <int VEC>
__global__ void __launch_bounds__(256)
min_pool_backward_kernel(const float* __restrict__ gy, const int32_t* __restrict__ arg, float* __restrict__ dx,
                         int H, int W, int C, int Kh, int Kw, int Sh, int Sw, int pad_top, int pad_left, int Nh,
                         int Nw, FastDiv by_c, FastDiv by_sw) {
    const unsigned e = (blockIdx.y * 256u + threadIdx.x) * VEC;
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
    float sum[VEC];
#pragma unroll
    for (int v = 0; v < VEC; ++v) sum[v] = 0.0f;
    for (int nh = nh_hi; nh >= nh_lo; --nh) {
        const int kh = hp - nh * Sh;
        for (int nw = nw_hi; nw >= nw_lo; --nw) {
            const int pos = kh * Kw + (wp - nw * Sw);
            const size_t o = (((size_t)b * Nh + nh) * Nw + nw) * C + c;
            // both values are requested at once: a gradient fetched only after the position has
            // been looked at would cost a second trip to memory
            int where[VEC];
            float g[VEC];
            if (VEC == 4) {
                const int4 a4 = *reinterpret_cast<const int4*>(arg + o);
                const float4 g4 = *reinterpret_cast<const float4*>(gy + o);
                where[0] = a4.x; where[1] = a4.y; where[2] = a4.z; where[3] = a4.w;
                g[0] = g4.x; g[1] = g4.y; g[2] = g4.z; g[3] = g4.w;
            } else {
                where[0] = arg[o];
                g[0] = gy[o];
            }
#pragma unroll
            for (int v = 0; v < VEC; ++v) sum[v] += where[v] == pos ? g[v] : 0.0f;
        }
    }
    float* out = dx + (size_t)row * W * C + e;
    if (VEC == 4) *reinterpret_cast<float4*>(out) = make_float4(sum[0], sum[1], sum[2], sum[3]);
    else *out = sum[0];
}

// xpad[b, hp, wp, c] = x[b, hp - top, wp - left, c] inside the image, `value` outside.
// blockIdx.x = padded row (b, hp); VEC floats per thread (VEC = 4 when C is a multiple of 4 and both
// tensors are 16-byte aligned: a group of four then never straddles a pixel).
template <int VEC>
__global__ void __launch_bounds__(256)
pad_time_kernel(const float* __restrict__ x, float* __restrict__ xpad, int H, int W, int C, int top, int left,
                int Hp, int Wp, float value, FastDiv by_c) {
    const unsigned e = (blockIdx.y * 256u + threadIdx.x) * VEC;            // (wp, c) within the padded row
    if (e >= (unsigned)(Wp * C)) return;
    const unsigned b = blockIdx.x / (unsigned)Hp;
    const int hp = (int)(blockIdx.x - b * (unsigned)Hp);
    const int wp = (int)fast_div(e, by_c), c = (int)e - wp * C;
    const int h = hp - top, w = wp - left;
    const bool inside = h >= 0 && h < H && w >= 0 && w < W;
    float* out = xpad + (size_t)blockIdx.x * Wp * C + e;
    const float* in = x + (((size_t)b * H + (inside ? h : 0)) * W + (inside ? w : 0)) * C + c;
    if (VEC == 4) {
        float4 v = make_float4(value, value, value, value);
        if (inside) v = *reinterpret_cast<const float4*>(in);
        *reinterpret_cast<float4*>(out) = v;
    } else {
        *out = inside ? *in : value;
    }
}

// dx[b, h, w, c] = dxpad[b, h + top, w + left, c]
template <int VEC>
__global__ void __launch_bounds__(256)
crop_time_kernel(const float* __restrict__ dxpad, float* __restrict__ dx, int H, int W, int C, int top, int left,
                 int Hp, int Wp) {
    const unsigned e = (blockIdx.y * 256u + threadIdx.x) * VEC;            // (w, c) within the row
    if (e >= (unsigned)(W * C)) return;
    const unsigned b = blockIdx.x / (unsigned)H;
    const int h = (int)(blockIdx.x - b * (unsigned)H);
    const float* in = dxpad + (((size_t)b * Hp + h + top) * Wp + left) * C + e;
    float* out = dx + (size_t)blockIdx.x * W * C + e;
    if (VEC == 4) *reinterpret_cast<float4*>(out) = *reinterpret_cast<const float4*>(in);
    else *out = *in;
}

}  // namespace

int launch_pad_time(const float* x, float* xpad, const PadGeom& g, float value, hipStream_t stream) {
    const int64_t rows = g.B * g.Hp, per_row = g.Wp * g.C;
    if (rows <= 0 || per_row <= 0) return SNNTC_OK;
    const bool vec = g.C % 4 == 0 && ((uintptr_t)x % 16 == 0) && ((uintptr_t)xpad % 16 == 0);
    const int64_t threads = vec ? per_row / 4 : per_row;
    dim3 grid((unsigned)rows, (unsigned)((threads + 255) / 256));
    if (grid.y > 65535u) return fail(SNNTC_ERR_TOO_LARGE, "padding: row of %lld elements too long", (long long)per_row);
    {
        KernelTimerScope timer_("pad_time", stream);
        const FastDiv by_c = make_fast_div(g.C, per_row);
        if (vec)
            hipLaunchKernelGGL(pad_time_kernel<4>, grid, dim3(256), 0, stream, x, xpad, (int)g.H, (int)g.W, (int)g.C,
                               (int)g.top, (int)g.left, (int)g.Hp, (int)g.Wp, value, by_c);
        else
            hipLaunchKernelGGL(pad_time_kernel<1>, grid, dim3(256), 0, stream, x, xpad, (int)g.H, (int)g.W, (int)g.C,
                               (int)g.top, (int)g.left, (int)g.Hp, (int)g.Wp, value, by_c);
    }
    SNNTC_HIP_CHECK(hipGetLastError());
    return SNNTC_OK;
}

int launch_crop_time(const float* dxpad, float* dx, const PadGeom& g, hipStream_t stream) {
    const int64_t rows = g.B * g.H, per_row = g.W * g.C;
    if (rows <= 0 || per_row <= 0) return SNNTC_OK;
    // a group of four starts at ((..) * Wp + left) * C + e floats: a multiple of 4 when C is
    const bool vec = g.C % 4 == 0 && ((uintptr_t)dx % 16 == 0) && ((uintptr_t)dxpad % 16 == 0);
    const int64_t threads = vec ? per_row / 4 : per_row;
    dim3 grid((unsigned)rows, (unsigned)((threads + 255) / 256));
    if (grid.y > 65535u) return fail(SNNTC_ERR_TOO_LARGE, "padding: row of %lld elements too long", (long long)per_row);
    {
        KernelTimerScope timer_("crop_time", stream);
        if (vec)
            hipLaunchKernelGGL(crop_time_kernel<4>, grid, dim3(256), 0, stream, dxpad, dx, (int)g.H, (int)g.W, (int)g.C,
                               (int)g.top, (int)g.left, (int)g.Hp, (int)g.Wp);
        else
            hipLaunchKernelGGL(crop_time_kernel<1>, grid, dim3(256), 0, stream, dxpad, dx, (int)g.H, (int)g.W, (int)g.C,
                               (int)g.top, (int)g.left, (int)g.Hp, (int)g.Wp);
    }
    SNNTC_HIP_CHECK(hipGetLastError());
    return SNNTC_OK;
}

static bool aligned16(const void* p) { return (uintptr_t)p % 16 == 0; }

int launch_min_pool_forward(const float* x, float* y, int32_t* arg, const PoolGeom& g, float pad_value,
                            const TimeCopy& copy, hipStream_t stream) {
    const int64_t rows = g.B * g.Nh, per_row = g.Nw * g.C;
    if (rows <= 0 || per_row <= 0) return SNNTC_OK;
    const bool vec = g.C % 4 == 0 && aligned16(x) && aligned16(y) && aligned16(arg) && aligned16(copy.dst);
    const int64_t threads = vec ? per_row / 4 : per_row;
    dim3 grid((unsigned)rows, (unsigned)((threads + 255) / 256));
    if (grid.y > 65535u) return fail(SNNTC_ERR_TOO_LARGE, "pooling: output row of %lld elements too long", (long long)per_row);
    {
        KernelTimerScope timer_("min_pool", stream);
        auto kern = vec ? min_pool_forward_kernel<4> : min_pool_forward_kernel<1>;
        hipLaunchKernelGGL(kern, grid, dim3(256), 0, stream, x, y, arg, (int)g.H, (int)g.W, (int)g.C, (int)g.Kh,
                           (int)g.Kw, (int)g.Sh, (int)g.Sw, (int)g.pad_top, (int)g.pad_left, (int)g.Nh, (int)g.Nw,
                           pad_value, make_fast_div(g.C, per_row), copy);
    }
    SNNTC_HIP_CHECK(hipGetLastError());
    return SNNTC_OK;
}

int launch_min_pool_backward(const float* gy, const int32_t* arg, float* dx, const PoolGeom& g, hipStream_t stream) {
    const int64_t rows = g.B * g.H, per_row = g.W * g.C;
    if (rows <= 0 || per_row <= 0) return SNNTC_OK;
    const bool vec = g.C % 4 == 0 && aligned16(gy) && aligned16(arg) && aligned16(dx);
    const int64_t threads = vec ? per_row / 4 : per_row;
    dim3 grid((unsigned)rows, (unsigned)((threads + 255) / 256));
    if (grid.y > 65535u) return fail(SNNTC_ERR_TOO_LARGE, "pooling: input row of %lld elements too long", (long long)per_row);
    {
        KernelTimerScope timer_("min_pool_grad", stream);
        auto kern = vec ? min_pool_backward_kernel<4> : min_pool_backward_kernel<1>;
        hipLaunchKernelGGL(kern, grid, dim3(256), 0, stream, gy, arg, dx, (int)g.H, (int)g.W, (int)g.C, (int)g.Kh,
                           (int)g.Kw, (int)g.Sh, (int)g.Sw, (int)g.pad_top, (int)g.pad_left, (int)g.Nh, (int)g.Nw,
                           make_fast_div(g.C, per_row), make_fast_div(g.Sw, g.W + g.Kw + g.Sw));
    }
    SNNTC_HIP_CHECK(hipGetLastError());
    return SNNTC_OK;
}

}  // namespace snntc
