// Shared declarations of the gfx950 SNN-TC library: status plumbing, the parsed form of the two
// params vectors, conv geometry and the launcher prototypes that api.hip chains together.
#pragma once

#include <hip/hip_runtime.h>
#include <math.h>
#include <stddef.h>
#include <stdint.h>

#include "../../include/snntc.h"

namespace snntc {

constexpr int kWave = 64;              // CDNA wavefront width
constexpr int kMaxSegment = 8192;      // longest segment one sorting network takes; longer ones are merged from pieces
constexpr int kMaxLongSegment = 1 << 24;
constexpr size_t kAlign = 256;         // workspace sub-buffer alignment
constexpr int kMaxDevices = 64;        // device indices the per-device one-time state covers

// Records a formatted message for snntc_last_error() and returns `code`.
int fail(int code, const char* fmt, ...);

#define SNNTC_HIP_CHECK(expr)                                                              \
    do {                                                                                   \
        hipError_t e_ = (expr);                                                            \
        if (e_ != hipSuccess)                                                              \
            return ::snntc::fail(SNNTC_ERR_HIP, "%s failed: %s", #expr, hipGetErrorString(e_)); \
    } while (0)

inline size_t align_up(size_t v) { return (v + kAlign - 1) / kAlign * kAlign; }

// Workgroups are handed to the eight XCDs (each with an L2 of its own) round-robin by workgroup
// id.  xcd_contiguous() renumbers a 1-D grid so that every XCD works on one contiguous range of
// the returned ids: neighbours in that numbering, which share operands, then share an L2 too.
// A bijection on [0, total) for any total.
constexpr int kXcds = 8;
__device__ __forceinline__ int xcd_contiguous(int block, int total) {
    const int xcd = block % kXcds, local = block / kXcds;
    const int per = total / kXcds, extra = total % kXcds;
    return xcd * per + (xcd < extra ? xcd : extra) + local;
}

// The instruction arbiter of a SIMD prefers its oldest wavefront.  Wavefronts that start together
// on long loops of equal length therefore do not advance together: the oldest runs at the pace of a
// lone wavefront, the youngest crawls, and once the older ones are gone the SIMD is left with one
// or two wavefronts that cannot fill it.  rotate_wave_priority(turn) gives the wavefronts of a SIMD
// the top priority in turns: called with a wave-uniform counter that advances at the same pace in
// all of them (a loop iteration count) plus a number that differs between the wavefronts of a SIMD
// (wavefronts of a workgroup go to the four SIMDs round-robin, so index / 4 does), it keeps their
// progress level, and they finish together.  s_setprio takes its level as an immediate.
__device__ __forceinline__ void rotate_wave_priority(int turn) {
    switch (turn & 3) {
        case 0: __builtin_amdgcn_s_setprio(0); break;
        case 1: __builtin_amdgcn_s_setprio(1); break;
        case 2: __builtin_amdgcn_s_setprio(2); break;
        default: __builtin_amdgcn_s_setprio(3); break;
    }
}

// Opt-in per-kernel timing (snntc_profile_*): while enabled, every launcher brackets its kernel
// with a pair of HIP events on the launch stream.  Disabled (the default) it costs one branch.
struct KernelTimerScope {
    KernelTimerScope(const char* name, hipStream_t stream);
    ~KernelTimerScope();
    int slot;
    hipStream_t stream;
};

// The scalar knobs every kernel needs, taken from either params layout.
struct NeuronParams {
    float max_time;   // MAX_SPIKE_TIME
    float max_cmp;    // MAX_SPIKE_TIME - 0.1 evaluated in fp32 (snntc/snnfc_kernels.cu.cc:27)
    float theta;      // Spike_Threshold
    float biasvolt;   // input value of the bias row
    int bias;         // biasvolt > 1e-8
    int wait_polls;   // scan_lds_split_kernel: polls a tester wavefront spends on the producer's sums before it
                      // gives up (set by the scan launcher, see scan_wait_polls)
};

// The weight-gradient kernels add up u * min(x - y, 0) over the segments.  They evaluate the second
// factor as -clamp01((y - x) * s) / s with s a power of two: fma(x, -s, y*s) rounds exactly like
// the difference itself, the [0, 1] clamp is an output modifier of the fma, and the factor -1/s is
// applied once to the finished sum, so the result has the bits of the plain sub / min / fma
// sequence at two vector instructions per term instead of three.  1/s is the power of two above
// 2 * MAX_SPIKE_TIME: the clamp's upper end is never reached while inputs stay above
// -MAX_SPIKE_TIME (outputs that take part are below MAX_SPIKE_TIME by construction).
struct LeadScale {
    float neg_s;      // -s
    float post;       // -1/s
};
inline LeadScale lead_scale(float max_time) {
    int e = 0;
    if (max_time > 1.0f) {
        if (max_time < 3e28f) frexpf(max_time, &e);      // max_time < 2^e
        else e = 95;
    }
    return LeadScale{-ldexpf(1.0f, -(e + 1)), -ldexpf(1.0f, e + 1)};
}
__device__ __forceinline__ float scaled_lead(float x, float neg_s, float ys) {
    return __builtin_amdgcn_fmed3f(__fmaf_rn(x, neg_s, ys), 0.0f, 1.0f);
}

// Where a segment's elements come from: rows of a dense matrix, or patches of an NHWC image
// gathered on the fly (patch s=(a*Nh+nh)*Nw+nw, element i=(kh*Kw+kw)*C+c).
struct SegmentSource {
    const float* base;
    int conv;         // 0: dense rows of length I;  1: implicit im2col
    int I;            // segment length (dense in_size or Kh*Kw*C)
    int H, W, C, Kh, Kw, Sh, Sw, Nh, Nw;
};

struct ConvGeom {
    int64_t B, H, W, C, Kc, Kh, Kw, Sh, Sw, Nh, Nw, P, S;
};

// Optional second destination of the spike times a scan writes: an NHWC image tensor [*, h, w, J]
// in which segment s = (a * Nh + nh) * Nw + nw is pixel (nh + top, nw + left) of image a -- the
// padded input of the next layer, whose border the caller has filled.  dst == NULL: none.
struct TimeCopy {
    float* dst;
    int Nh, Nw, h, w, top, left;
};
__device__ __forceinline__ size_t time_copy_pixel(const TimeCopy& tc, int seg) {
    const int per_image = tc.Nh * tc.Nw;
    const int a = seg / per_image, r = seg - a * per_image;
    const int nh = r / tc.Nw, nw = r - nh * tc.Nw;
    return ((size_t)a * tc.h + nh + tc.top) * tc.w + nw + tc.left;
}

// The window of the padded input's gradient that conv dX stores:
// dx[B, h, w, C] = dxpad[:, top : top + h, left : left + w, :] (the whole of it: {H, W, 0, 0}).
struct CropGeom {
    int h, w, top, left;
};

// ---- launchers (each enqueues on `stream` and returns a status) --------------------------------

// Row stride of the sorted / perm scratch arrays: segments are padded to a multiple of 16 entries
// so the scan can fetch them in aligned groups without bounds checks.
inline int64_t padded_stride(int64_t I) { return (I + 15) / 16 * 16; }

// Segmented stable ascending sort: sorted[S,out_stride] and perm[S,out_stride] (entries past the
// segment length hold +inf / 0), n_real[S] = number of values <= max_cmp (may be NULL).
// Segments longer than kMaxSegment are sorted in pieces and merged in global memory; they need
// `long_ws`, sort_long_workspace_bytes(S, I) bytes of scratch (NULL otherwise).
size_t sort_long_workspace_bytes(int64_t S, int64_t I);
int launch_sort(const SegmentSource& src, int64_t S, float* sorted, int32_t* perm, int32_t* n_real,
                int out_stride, float max_cmp, void* long_ws, hipStream_t stream);

// Conv patch sort by merging pre-sorted pixels (merge.hip): pix_z / pix_c are the [B*H*W, Cs] outputs
// of launch_sort on the image's pixels.
bool merge_sort_supported(const ConvGeom& g);
int launch_merge_patches(const float* pix_z, const int32_t* pix_c, int64_t Cs, float* sorted, int32_t* perm,
                         int32_t* n_real, const ConvGeom& g, int64_t stride, float max_cmp, hipStream_t stream);

// Copies the first I entries of every padded row into dense [S,I] arrays (either may be NULL).
int launch_unpad_rows(const float* sorted, const int32_t* perm, float* sorted_out, int32_t* perm_out,
                      int64_t S, int64_t I, int64_t stride, hipStream_t stream);

// Causal-set scan over sorted segments (rows of length `stride`, n_real inputs each):
// y[S,J], rcp[S,J], optional causal_k[S,J].
int launch_scan(const float* sorted, const int32_t* perm, const int32_t* n_real, const float* w, float* y,
                float* rcp, int32_t* causal_k, int64_t S, int64_t I, int64_t stride, int64_t J,
                const NeuronParams& np, const TimeCopy& copy, hipStream_t stream);

// Bounded wait of the classifier-head scan (scan_lds_split_kernel): the poll limit launches use from now on
// (polls < 0 restores the default), and the number of tester wavefronts that ran out of it on the current
// device since the process started (read with a copy on `stream` and a wait for that stream).
void set_scan_wait_polls(int polls);
int read_scan_giveups(int64_t* count, hipStream_t stream);

// One-time set-up on device `dev`, which must be the current device: the dynamic-LDS limits of every
// scan / merge instantiation (and the CU count the scan sizes its launches with).  The launchers call
// them on their first use of a device; snntc_init() calls them ahead of time.
int scan_prepare_device(int dev, int* cu_count_out);
int merge_prepare_device(int dev);

// upm = valid ? grad*rcp : 0   (valid: y <= MAX-0.1; n elements), and, in the same launch, the weight copy dX reads from: mode 0 none, mode 1
// wt[cols, rows] = w[rows, cols]^T, mode 2 the regrouped copy of a conv layer's weights
// (wt[tap][cols / 4][chan][cols % 4] from w[(tap, chan), cols], rows = taps * chan).  `zeros`, if not
// NULL, are n_zeros (<= 256) floats the launch clears: the op's all-zero dParams output.
int launch_backward_prologue(const float* grad, const float* y, const float* rcp, float* upm, int64_t n, const NeuronParams& np, int mode, const float* w, float* wt, int64_t rows,
                             int64_t cols, int64_t chan, float* zeros, int n_zeros, hipStream_t stream);

int launch_fc_grad_input(const float* x, const float* wt, const float* upm, const float* ym, float* dx,
                         int64_t B, int64_t I, int64_t J, int64_t wt_stride, hipStream_t stream);

// dW for dense rows or implicit patches.  The segment range may be cut into `nsplit` slices whose
// partial sums (scratch `dst`, nsplit x rows x J) are added in slice order by launch_reduce_partials.
int weight_grad_splits(int64_t S, int64_t base_blocks);
int grad_weight_blocks(int64_t rows, int64_t J);
int launch_grad_weight_rows(const SegmentSource& src, const float* upm, const float* ym, float* dst,
                            int nsplit, int64_t S, int64_t J, int64_t row_start, const NeuronParams& np,
                            hipStream_t stream);
int launch_reduce_partials(const float* partial, float* dw, int64_t n, int nsplit, hipStream_t stream);

// Dense layers with at most 16 outputs: masked upstream values, dX and dW in one launch (dx / dw
// may be NULL).  `partial` (fc_backward_narrow_splits(B) x rows x J floats) is used when the batch
// spans more than one block of samples.
bool fc_backward_narrow_supported(int64_t J);
int fc_backward_narrow_splits(int64_t B);
int launch_fc_backward_narrow(const float* x, const float* w, const float* grad, const float* y, const float* rcp,
                              float* dx, float* dw, float* partial, float* zeros, int n_zeros, int64_t B, int64_t I,
                              int64_t J, const NeuronParams& np, hipStream_t stream);

// Conv layers with many channels: lane = channel (dX) / wide row blocks (dW), see cv_grad.hip.
bool cv_grad_input_chan_supported(const ConvGeom& g);
// launch_cv_grad_input_chan reads the weights from the copy regrouped by launch_backward_prologue (mode 2).
int launch_cv_grad_input_chan(const float* xpad, const float* wq, const float* upm, const float* ym,
                              float* dx, const CropGeom& crop, const ConvGeom& g, const NeuronParams& np,
                              hipStream_t stream);
bool cv_grad_weight_wide_supported(const ConvGeom& g);
int cv_grad_weight_wide_blocks(const ConvGeom& g);
int launch_cv_grad_weight_wide(const float* xpad, const float* upm, const float* ym, float* dst, int nsplit,
                               const ConvGeom& g, int64_t rows, const NeuronParams& np, hipStream_t stream);

// Conv dX for layers launch_cv_grad_input_chan does not take; dxp is scratch of S * P floats.
int launch_cv_grad_input(const SegmentSource& src, const float* wt, const float* upm, const float* ym, float* dxp,
                         float* dx, const CropGeom& crop, const ConvGeom& g, int64_t wt_stride, hipStream_t stream);

int launch_fill_zero(float* p, int64_t n, hipStream_t stream);

// Earliest-spike pooling (pool.hip).  Window (nh, nw) starts at pixel (nh*Sh - pad_top, nw*Sw - pad_left);
// pixels outside the image count as pad_value.  arg (may be NULL in the forward pass) records kh*Kw+kw
// of the first window position that attains the minimum.
struct PoolGeom {
    int64_t B, H, W, C, Kh, Kw, Sh, Sw, pad_top, pad_left, Nh, Nw;
};
int launch_min_pool_forward(const float* x, float* y, int32_t* arg, const PoolGeom& g, float pad_value,
                            const TimeCopy& copy, hipStream_t stream);
int launch_min_pool_backward(const float* gy, const int32_t* arg, float* dx, const PoolGeom& g, hipStream_t stream);

// SAME padding of a conv layer's input with a constant (pool.hip): xpad[B,Hp,Wp,C] holds x[B,H,W,C]
// at row offset top, column offset left, `value` elsewhere; launch_crop_time is the reverse copy.
struct PadGeom {
    int64_t B, H, W, C, top, left, Hp, Wp;
};
int launch_pad_time(const float* x, float* xpad, const PadGeom& g, float value, hipStream_t stream);
int launch_crop_time(const float* dxpad, float* dx, const PadGeom& g, hipStream_t stream);

// w[t] -= lr * dw[t] for `count` tensors of n[t] elements (host arrays of device pointers).
int launch_sgd_update(float* const* w, const float* const* dw, const int64_t* n, int count, float lr,
                      hipStream_t stream);
int launch_softmax_time_loss(const float* times, const float* label, float* sample_loss, float* dtimes,
                             int64_t B, int64_t J, hipStream_t stream);

}  // namespace snntc
