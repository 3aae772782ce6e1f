// Backward kernels of the dense and conv SNN-TC layers.
//
// Contract (snntc/snnfcgrad_kernels.cu.cc:60,118-120,159-173; snntc/snncvgrad_kernels.cu.cc:71,143,
// 190-204), with up = grad[:S] * oldout[S:], MAXc = MAX_SPIKE_TIME - 0.1:
//   dX[s,i] = sum_j [x_si <= y_sj and y_sj <= MAXc] up_sj * W[i,j]
//   dW[i,j] = sum_s [x_si <= MAXc and y_sj <= MAXc and x_si <= y_sj] (x_si - y_sj) * up_sj
//   dW[I,j] = the same with x = biasvolt (bias row)
// For the conv layer s runs over output pixels and x_si is gathered from the padded image; dX is
// accumulated in gather form (every input pixel sums over the output pixels whose window covers
// it), so no atomics are needed and the result does not depend on scheduling.
//
// The validity test on y is folded into one array prepared once per call,
//   upm = valid ? up : 0,
// so that a term of an output that takes no part vanishes whatever its mask says (the kernels read y
// itself, under the parameter name ym); the weight-gradient mask is folded into arithmetic: for x <= y the term (x-y) is <= 0 and
// for x > y it is > 0, hence [x <= y](x - y) == min(x - y, 0).
#include "snntc_common.h"

namespace snntc {
namespace {

// First launch of a backward pass.  The elementwise pass over the layer's outputs,
//   upm = valid ? grad * rcp : 0   (valid: y <= MAX - 0.1),
// and the weight copy dX reads from do not depend on each other: one launch does both, the first
// prep_blocks workgroups the former, the rest the latter.
//   mode 1: wt[cols, rows] = w[rows, cols]^T, a 32 x 32 tile per workgroup
//   mode 2: w[(tap, c), kc] -> wt[tap][kc / 4][c][kc % 4], one 16-byte piece per thread (cols = Kc, a
//           multiple of 4; chan = C)
__global__ void __launch_bounds__(256)
backward_prologue_kernel(const float* __restrict__ grad, const float* __restrict__ y,
                         const float* __restrict__ rcp, float* __restrict__ upm, int64_t n, float max_cmp,
                         int prep_blocks, int vec4, int mode, const float* __restrict__ w,
                         float* __restrict__ wt, int rows, int cols, int chan, float* __restrict__ zeros,
                         int n_zeros) {
    __shared__ float tile[32][33];
    if (blockIdx.x == 0 && (int)threadIdx.x < n_zeros) zeros[threadIdx.x] = 0.0f;    // the dParams output
    if ((int)blockIdx.x < prep_blocks) {
        const int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
        if (vec4) {                                      // n a multiple of 4, the arrays 16-byte aligned
            if (4 * t >= n) return;
            const float4 yv = reinterpret_cast<const float4*>(y)[t], gv = reinterpret_cast<const float4*>(grad)[t];
            const float4 rv = reinterpret_cast<const float4*>(rcp)[t];
            float4 u;
            u.x = yv.x <= max_cmp ? gv.x * rv.x : 0.0f;
            u.y = yv.y <= max_cmp ? gv.y * rv.y : 0.0f;
            u.z = yv.z <= max_cmp ? gv.z * rv.z : 0.0f;
            u.w = yv.w <= max_cmp ? gv.w * rv.w : 0.0f;
            reinterpret_cast<float4*>(upm)[t] = u;
            return;
        }
        if (t >= n) return;
        const float yv = y[t];
        const bool valid = yv <= max_cmp;
        upm[t] = valid ? grad[t] * rcp[t] : 0.0f;
        return;
    }
    const int blk = (int)blockIdx.x - prep_blocks;
    if (mode == 1) {
        const int tiles_x = (cols + 31) / 32;
        const int tx = threadIdx.x % 32, ty = threadIdx.x / 32;       // 32 x 8
        const int c0 = (blk % tiles_x) * 32, r0 = (blk / tiles_x) * 32;
        for (int dy = ty; dy < 32; dy += 8) {
            const int r = r0 + dy, c = c0 + tx;
            tile[dy][tx] = (r < rows && c < cols) ? w[(size_t)r * cols + c] : 0.0f;
        }
        __syncthreads();
        for (int dy = ty; dy < 32; dy += 8) {
            const int c = c0 + dy, r = r0 + tx;
            if (r < rows && c < cols) wt[(size_t)c * rows + r] = tile[tx][dy];
        }
    } else {
        const int k4 = cols / 4;
        const int64_t t = (int64_t)blk * blockDim.x + threadIdx.x;    // over (tap, c, kc / 4), kc / 4 fastest
        if (t >= (int64_t)rows * k4) return;
        const int64_t row = t / k4;                                   // tap * C + c
        const int q = (int)(t - row * k4);
        const int64_t tap = row / chan;
        const int c = (int)(row - tap * chan);
        reinterpret_cast<float4*>(wt)[(tap * k4 + q) * chan + c] = reinterpret_cast<const float4*>(w)[t];
    }
}

__global__ void __launch_bounds__(256) fill_zero_kernel(float* __restrict__ p, int64_t n) {
    const int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (t < n) p[t] = 0.0f;
}

// Source offset of weight row e relative to the segment base (dense: the column; conv: kh/kw/c).
__device__ __forceinline__ int row_offset(const SegmentSource& src, int e) {
    if (!src.conv) return e;
    const int span = src.Kw * src.C;
    const int kh = e / span;
    return kh * src.W * src.C + (e - kh * span);
}

// Base of segment s inside the source tensor.
__device__ __forceinline__ const float* segment_base(const SegmentSource& src, int s) {
    if (!src.conv) return src.base + (size_t)s * src.I;
    const int per_img = src.Nh * src.Nw;
    const int a = s / per_img, r2 = s - a * per_img;
    const int nh = r2 / src.Nw, nw = r2 - nh * src.Nw;
    return src.base + ((size_t)(a * src.H + nh * src.Sh) * src.W + (size_t)nw * src.Sw) * src.C;
}

// ---------------------------------------------------------------------------------------------
// Dense dX.  Lanes run across inputs i (wt[j, i] is read coalesced), each thread carries RB
// samples whose y/up values are wave-uniform; the four wavefronts of a block split the j range
// and are summed through LDS in a fixed order.
// ---------------------------------------------------------------------------------------------
constexpr int DX_RB = 4;
constexpr int DX_STEP = 4;

// PATCHES: the "samples" are the implicit patches of a conv layer (src.conv) and the result is the
// gradient per patch element, dx[S, P], which cv_col2im_kernel then folds back onto the image.
template <bool PATCHES>
__global__ void __launch_bounds__(256)
fc_grad_input_kernel(const SegmentSource src, const float* __restrict__ wt,
                     const float* __restrict__ upm, const float* __restrict__ ym, float* __restrict__ dx,
                     int B, int I, int J, int wt_stride) {
    const float* __restrict__ x = src.base;
    __shared__ float red[3][DX_RB][kWave];
    const int lane = threadIdx.x % kWave;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
    const int i = blockIdx.y * kWave + lane;
    const unsigned ic = (unsigned)min(i, I - 1);
    const int b0 = blockIdx.x * DX_RB;

    float xr[DX_RB], acc[DX_RB];
    // the y / up rows of the block's samples: one base pointer each and a byte offset per sample (eight
    // scalar registers instead of sixteen for eight pointers; samples past the batch repeat the last row)
    const float* __restrict__ ybase = ym + (size_t)b0 * J;
    const float* __restrict__ ubase = upm + (size_t)b0 * J;
    int row_bytes[DX_RB];
#pragma unroll
    for (int r = 0; r < DX_RB; ++r) {
        const int brow = min(b0 + r, B - 1);
        xr[r] = PATCHES ? segment_base(src, brow)[row_offset(src, (int)ic)] : x[(size_t)brow * I + ic];
        row_bytes[r] = (brow - b0) * J * (int)sizeof(float);
        acc[r] = 0.0f;
    }
    const int jq = (J + 3) / 4;
    const int j_lo = wave * jq, j_hi = min(J, j_lo + jq);
    const float* __restrict__ wcol = wt + ic;
    int j = j_lo;
    // DX_STEP columns at a time.  The y / up values of the block's samples are wave-uniform and arrive
    // through the scalar path; scalar loads return in no fixed order, so a wavefront can only wait for
    // all of them, and a load issued right before its use costs a round trip every time.  The loop
    // therefore runs one step ahead: wait for the values of this step (requested a step ago), request
    // those of the next into the other set of registers, then do this step's arithmetic.  The
    // weights (vector loads, which return in order) run one step ahead as well.
    {
        typedef float f4 __attribute__((ext_vector_type(4)));
        auto request = [&](f4 (&yv)[DX_RB], f4 (&uv)[DX_RB], int jj) {
            const int off = jj * (int)sizeof(float);
#pragma unroll
            for (int r = 0; r < DX_RB; ++r) {
                const int o = row_bytes[r] + off;
                asm volatile("s_load_dwordx4 %0, %1, %2" : "=s"(yv[r]) : "s"(ybase), "s"(o));
                asm volatile("s_load_dwordx4 %0, %1, %2" : "=s"(uv[r]) : "s"(ubase), "s"(o));
            }
        };
        auto arrived = [&](f4 (&yv)[DX_RB], f4 (&uv)[DX_RB]) {
            asm volatile("s_waitcnt lgkmcnt(0)"
                         : "+s"(yv[0]), "+s"(yv[1]), "+s"(yv[2]), "+s"(yv[3]), "+s"(uv[0]), "+s"(uv[1]), "+s"(uv[2]),
                           "+s"(uv[3]));
        };
        auto weights = [&](float (&wv)[DX_STEP], int jj) {
#pragma unroll
            for (int u = 0; u < DX_STEP; ++u) wv[u] = (wt + (size_t)(jj + u) * wt_stride)[ic];
        };
        // acc[r] += up * w where x <= y; the others are skipped, as in the reference
        // (snnfcgrad_kernels.cu.cc:60), not added as zeros.  (Writing the compare into EXEC and running
        // the multiply-add under it saves the select but no time: the EXEC round trip stalls the issue.)
        auto macs = [&](const f4 (&yv)[DX_RB], const f4 (&uv)[DX_RB], const float (&wv)[DX_STEP]) {
#pragma unroll
            for (int r = 0; r < DX_RB; ++r) {
#pragma unroll
                for (int u = 0; u < DX_STEP; ++u)
                    acc[r] = xr[r] <= yv[r][u] ? __fmaf_rn(uv[r][u], wv[u], acc[r]) : acc[r];
            }
        };
        static_assert(DX_RB == 4 && DX_STEP == 4, "register sets of the pipelined loop");
        const int steps = (j_hi - j_lo) / DX_STEP;
        if (steps > 0) {
            f4 ya[DX_RB], ua[DX_RB], yb[DX_RB], ub[DX_RB];
            float wa[DX_STEP], wb[DX_STEP];
            const int j_last = j_lo + (steps - 1) * DX_STEP;      // requests past the last step re-read it
            request(ya, ua, j);
            weights(wa, j);
            for (int sidx = 0; sidx + 2 <= steps; sidx += 2) {
                const int jn = j + DX_STEP, jnn = min(j + 2 * DX_STEP, j_last);
                arrived(ya, ua);
                request(yb, ub, jn);
                weights(wb, jn);
                __builtin_amdgcn_sched_barrier(0);                 // requests first, then the arithmetic
                macs(ya, ua, wa);
                __builtin_amdgcn_sched_barrier(0);
                arrived(yb, ub);
                request(ya, ua, jnn);
                weights(wa, jnn);
                __builtin_amdgcn_sched_barrier(0);
                macs(yb, ub, wb);
                __builtin_amdgcn_sched_barrier(0);
                j += 2 * DX_STEP;
            }
            arrived(ya, ua);                                       // nothing stays in flight
            if (steps & 1) macs(ya, ua, wa);
            j = j_lo + steps * DX_STEP;
        }
    }
    for (; j < j_hi; ++j) {
        const float wv = wcol[(size_t)j * wt_stride];
#pragma unroll
        for (int r = 0; r < DX_RB; ++r) {
            const int e = row_bytes[r] / (int)sizeof(float) + j;
            acc[r] = xr[r] <= ybase[e] ? __fmaf_rn(ubase[e], wv, acc[r]) : acc[r];
        }
    }
    if (wave > 0) {
#pragma unroll
        for (int r = 0; r < DX_RB; ++r) red[wave - 1][r][lane] = acc[r];
    }
    __syncthreads();
    if (wave == 0 && i < I) {
#pragma unroll
        for (int r = 0; r < DX_RB; ++r) {
            if (b0 + r < B)
                dx[(size_t)(b0 + r) * I + i] = ((acc[r] + red[0][r][lane]) + red[1][r][lane]) + red[2][r][lane];
        }
    }
}

// ---------------------------------------------------------------------------------------------
// dW for dense rows or implicit conv patches.  Lanes run across outputs j (y/up rows are read
// coalesced); each thread carries RI consecutive weight rows whose x values are wave-uniform.
// The segment range is cut into gridDim.z slices; a slice is further split over the four
// wavefronts of the block.  With more than one slice the per-slice sums go to `partial` and are
// added in slice order by reduce_partials_kernel.
// ---------------------------------------------------------------------------------------------
constexpr int DW_RI = 8;
constexpr int DW_UNROLL = 4;

__global__ void __launch_bounds__(256)
grad_weight_kernel(SegmentSource src, const float* __restrict__ upm, const float* __restrict__ ym,
                   float* __restrict__ dst, int S, int J, int rows, int row_start, int seg_per_slice,
                   float biasvolt, float neg_s, float post) {
    __shared__ float red[3][DW_RI][kWave];
    const int lane = threadIdx.x % kWave;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
    const int j = blockIdx.x * kWave + lane;
    const unsigned jc = (unsigned)min(j, J - 1);
    const int i0 = row_start + blockIdx.y * DW_RI;
    const int I = src.I;

    const int s_begin = blockIdx.z * seg_per_slice;
    const int s_end = min(S, s_begin + seg_per_slice);
    const int per_wave = (s_end - s_begin + 3) / 4;
    const int s_lo = s_begin + wave * per_wave;
    const int s_hi = min(s_end, s_lo + per_wave);

    float acc[DW_RI];
#pragma unroll
    for (int r = 0; r < DW_RI; ++r) acc[r] = 0.0f;
    const float* __restrict__ ycol = ym + jc;
    const float* __restrict__ ucol = upm + jc;

    // The RI weight rows of this block are contiguous in the source (always for dense rows, for
    // patches when the rows share one (kh, kw)): their x values come as one scalar fetch.
    const bool contiguous = i0 + DW_RI <= I && (!src.conv || (i0 % src.C) + DW_RI <= src.C);
    if (contiguous) {
        const int off0 = row_offset(src, i0);
        int s = s_lo;
        for (; s + DW_UNROLL <= s_hi; s += DW_UNROLL) {
            float yv[DW_UNROLL], uv[DW_UNROLL];
            const float* xb[DW_UNROLL];
#pragma unroll
            for (int u = 0; u < DW_UNROLL; ++u) {
                yv[u] = ycol[(size_t)(s + u) * J] * -neg_s;
                uv[u] = ucol[(size_t)(s + u) * J];
                xb[u] = segment_base(src, s + u) + off0;
            }
#pragma unroll
            for (int u = 0; u < DW_UNROLL; ++u) {
#pragma unroll
                for (int r = 0; r < DW_RI; ++r)
                    acc[r] = __fmaf_rn(scaled_lead(xb[u][r], neg_s, yv[u]), uv[u], acc[r]);
            }
        }
        for (; s < s_hi; ++s) {
            const float yv = ycol[(size_t)s * J] * -neg_s, uv = ucol[(size_t)s * J];
            const float* xb = segment_base(src, s) + off0;
#pragma unroll
            for (int r = 0; r < DW_RI; ++r) acc[r] = __fmaf_rn(scaled_lead(xb[r], neg_s, yv), uv, acc[r]);
        }
    } else {
        int off[DW_RI];
        bool is_bias[DW_RI];
#pragma unroll
        for (int r = 0; r < DW_RI; ++r) {
            const int i = min(i0 + r, rows - 1);
            is_bias[r] = i >= I;
            off[r] = row_offset(src, min(i, I - 1));
        }
        for (int s = s_lo; s < s_hi; ++s) {
            const float yv = ycol[(size_t)s * J] * -neg_s, uv = ucol[(size_t)s * J];
            const float* xb = segment_base(src, s);
#pragma unroll
            for (int r = 0; r < DW_RI; ++r) {
                const float xv = is_bias[r] ? biasvolt : xb[off[r]];
                acc[r] = __fmaf_rn(scaled_lead(xv, neg_s, yv), uv, acc[r]);
            }
        }
    }
    if (wave > 0) {
#pragma unroll
        for (int r = 0; r < DW_RI; ++r) red[wave - 1][r][lane] = acc[r];
    }
    __syncthreads();
    if (wave == 0 && j < J) {
        float* out = dst + (size_t)blockIdx.z * rows * J;
#pragma unroll
        for (int r = 0; r < DW_RI; ++r) {
            if (i0 + r < rows)
                out[(size_t)(i0 + r) * J + j] =
                    (((acc[r] + red[0][r][lane]) + red[1][r][lane]) + red[2][r][lane]) * post;
        }
    }
}

// ---------------------------------------------------------------------------------------------
// dW of a dense layer.  Same mapping as grad_weight_kernel (lane = output j, DW_RI weight rows per
// block, the block's samples shared out over its four wavefronts), arranged so that a wavefront
// waits for memory a few times instead of once per four samples -- at a batch of a few hundred
// samples the wavefronts are short-lived and there are too few of them to hide those waits:
//  * the x values of the block's rows, 256 samples at a time, are staged in LDS by all threads (the
//    tile after the current one is already on its way) and read back as broadcasts; rows past the
//    inputs read biasvolt, so the bias row needs no code of its own;
//  * the ym / upm values of DWD_BATCH samples are requested together before the first one is used.
// ---------------------------------------------------------------------------------------------
#ifndef SNNTC_DWD_BATCH
#define SNNTC_DWD_BATCH 16
#endif
constexpr int DWD_BATCH = SNNTC_DWD_BATCH;
constexpr int DWD_TILE = 256;                              // samples per staged tile: 64 per wavefront
static_assert(DW_RI == 8, "the staging below moves eight rows per sample");

__global__ void __launch_bounds__(256)
grad_weight_dense_kernel(const float* __restrict__ x, const float* __restrict__ upm, const float* __restrict__ ym,
                         float* __restrict__ dst, int S, int I, int J, int rows, int seg_per_slice, float biasvolt,
                         float neg_s, float post) {
    __shared__ __align__(16) float xt[2][DWD_TILE][DW_RI];
    __shared__ float red[3][DW_RI][kWave];
    const int lane = threadIdx.x % kWave;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
    const int j = blockIdx.x * kWave + lane;
    const unsigned jc = (unsigned)min(j, J - 1);
    const int i0 = blockIdx.y * DW_RI;
    const int s_begin = blockIdx.z * seg_per_slice;
    const int s_end = __builtin_amdgcn_readfirstlane(min(S, s_begin + seg_per_slice));
    // ym / upm of the slice through buffer descriptors: the sample's row is a scalar offset, the lane's
    // column a constant one, and no address is computed per lane (the launcher keeps a slice below 2 GB)
    const int slice_bytes = max(s_end - s_begin, 0) * J * (int)sizeof(float);
    const __amdgpu_buffer_rsrc_t ybuf =
        __builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(ym + (size_t)s_begin * J), 0, slice_bytes, 0x00020000);
    const __amdgpu_buffer_rsrc_t ubuf =
        __builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(upm + (size_t)s_begin * J), 0, slice_bytes, 0x00020000);
    const int col_bytes = (int)(jc * sizeof(float)), row_bytes = J * (int)sizeof(float);

    float acc[DW_RI];
#pragma unroll
    for (int r = 0; r < DW_RI; ++r) acc[r] = 0.0f;

    // element e = threadIdx.x + 256 * k of a tile: sample e / 8, row e % 8
    const int st_row = threadIdx.x % DW_RI;
    const int st_smp = threadIdx.x / DW_RI;                 // + 32 * k
    const bool st_input = i0 + st_row < I;
    const float* __restrict__ st_src = x + (st_input ? i0 + st_row : 0);
    float pending[DW_RI];
    auto fetch_tile = [&](int c0) {
#pragma unroll
        for (int k = 0; k < DW_RI; ++k) {
            const int s = min(c0 + st_smp + 32 * k, s_end - 1);
            pending[k] = st_input ? st_src[(size_t)s * I] : biasvolt;
        }
    };
    auto store_tile = [&](int buf) {
#pragma unroll
        for (int k = 0; k < DW_RI; ++k) xt[buf][st_smp + 32 * k][st_row] = pending[k];
    };

    // ym / upm of DWD_BATCH samples are requested together, then the batch is worked on.  (Requesting a
    // batch ahead of the arithmetic changes nothing: alone, the requests of a launch keep L2 busy for
    // about as long as the arithmetic keeps the vector units busy, and the two overlap only in part.)
    auto load_batch = [&](float (&yv)[DWD_BATCH], float (&uv)[DWD_BATCH], int sb) {
#pragma unroll
        for (int q = 0; q < DWD_BATCH; ++q) {
            const int sc = __builtin_amdgcn_readfirstlane(min(sb + q, s_end - 1));   // past the end: the last sample again
            const int off = (sc - s_begin) * row_bytes;
            yv[q] = __uint_as_float(__builtin_amdgcn_raw_buffer_load_b32(ybuf, col_bytes, off, 0));
            uv[q] = __uint_as_float(__builtin_amdgcn_raw_buffer_load_b32(ubuf, col_bytes, off, 0));
        }
    };
    auto run_batch = [&](const float (&yv)[DWD_BATCH], const float (&uv)[DWD_BATCH], int sb, int buf, int h) {
#pragma unroll
        for (int q = 0; q < DWD_BATCH; ++q) {
            const float4* xq = reinterpret_cast<const float4*>(&xt[buf][wave * (DWD_TILE / 4) + h + q][0]);
            const float4 xa = xq[0], xb = xq[1];
            const float xr[DW_RI] = {xa.x, xa.y, xa.z, xa.w, xb.x, xb.y, xb.z, xb.w};
            const float ys = yv[q] * -neg_s;
            const float u = sb + q < s_end ? uv[q] : 0.0f;  // the surplus of the last batch weighs nothing
#pragma unroll
            for (int r = 0; r < DW_RI; ++r) acc[r] = __fmaf_rn(scaled_lead(xr[r], neg_s, ys), u, acc[r]);
        }
    };

    if (s_begin < s_end) {
        fetch_tile(s_begin);
        store_tile(0);
        int buf = 0;
        for (int c0 = s_begin; c0 < s_end; c0 += DWD_TILE, buf ^= 1) {
            __syncthreads();                                // tile `buf` is complete; the other one is free
            const bool more = c0 + DWD_TILE < s_end;
            if (more) fetch_tile(c0 + DWD_TILE);
            const int w0 = c0 + wave * (DWD_TILE / 4);
#pragma unroll 1
            for (int h = 0; h < DWD_TILE / 4; h += DWD_BATCH) {
                const int sb = w0 + h;
                if (sb >= s_end) break;                     // wavefront-uniform
                float yv[DWD_BATCH], uv[DWD_BATCH];
                load_batch(yv, uv, sb);
                run_batch(yv, uv, sb, buf, h);
            }
            if (more) store_tile(buf ^ 1);
        }
    }
    if (wave > 0) {
#pragma unroll
        for (int r = 0; r < DW_RI; ++r) red[wave - 1][r][lane] = acc[r];
    }
    __syncthreads();
    if (wave == 0 && j < J) {
        float* out = dst + (size_t)blockIdx.z * rows * J;
#pragma unroll
        for (int r = 0; r < DW_RI; ++r) {
            if (i0 + r < rows)
                out[(size_t)(i0 + r) * J + j] =
                    (((acc[r] + red[0][r][lane]) + red[1][r][lane]) + red[2][r][lane]) * post;
        }
    }
}

// ---------------------------------------------------------------------------------------------
// Whole backward pass of a dense layer with few outputs (a classifier head: J <= 16) in one launch:
// the masked upstream values, dX and dW.  A wavefront covers 16 weight rows i (the bias row is one
// more row, with x = biasvolt and no dX) times four groups of JL adjacent columns: lane = (group,
// row).  A block takes up to NARROW_SAMPLES samples, whose scaled output times and upstream values
// it first puts into LDS; each of its wavefronts then walks every NARROW_WAVES-th sample.  dX[b, i]
// is complete after a sample -- the four column groups are added in the order (0 + 1) + (2 + 3) --
// and is stored at once; the dW sums of a lane run over the samples and are added across the
// wavefronts in wavefront order at the end.  Both inputs of the comparison x <= y are scaled by
// the same power of two, which does not change its outcome.  With more than one block of samples
// the dW sums go to `dst` as slices for reduce_partials_kernel.
// ---------------------------------------------------------------------------------------------
constexpr int NARROW_GROUPS = 4;
constexpr int NARROW_ROWS = kWave / NARROW_GROUPS;     // weight rows per block
constexpr int NARROW_JMAX = 4 * NARROW_GROUPS;
constexpr int NARROW_WAVES = 16;
constexpr int NARROW_SAMPLES = 256;

template <int JL>
__global__ void __launch_bounds__(NARROW_WAVES * kWave)
fc_backward_narrow_kernel(const float* __restrict__ x, const float* __restrict__ w,
                          const float* __restrict__ grad, const float* __restrict__ y,
                          const float* __restrict__ rcp, float* __restrict__ dx, float* __restrict__ dst,
                          int B, int I, int J, int rows, float max_cmp, float biasvolt, float neg_s, float post,
                          float* __restrict__ zeros, int n_zeros) {
    constexpr int JP = JL * NARROW_GROUPS;
    if (blockIdx.x == 0 && blockIdx.y == 0 && (int)threadIdx.x < n_zeros) zeros[threadIdx.x] = 0.0f;   // dParams
    // one more row than samples: (-inf, 0), which adds nothing, for the turns of a wavefront past
    // the block's last sample
    __shared__ float ys[NARROW_SAMPLES + 1][JP];           // scaled output time, -inf where masked out
    __shared__ float us[NARROW_SAMPLES + 1][JP];           // grad * 1/wsum, 0 where masked out
    __shared__ float red[NARROW_WAVES - 1][JL][kWave];
    const int lane = threadIdx.x % kWave;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
    const int group = lane / NARROW_ROWS;
    const int i = blockIdx.x * NARROW_ROWS + lane % NARROW_ROWS;
    const int j0 = group * JL;                             // first column of the lane
    const int b0 = blockIdx.y * NARROW_SAMPLES;
    const int n_s = min(NARROW_SAMPLES, B - b0);

    for (int e = threadIdx.x; e < n_s * JP; e += NARROW_WAVES * kWave) {
        const int bl = e / JP, j = e - bl * JP;
        float yv = -INFINITY, uv = 0.0f;
        if (j < J) {
            const size_t t = (size_t)(b0 + bl) * J + j;
            const float yt = y[t];
            if (yt <= max_cmp) { yv = yt * -neg_s; uv = grad[t] * rcp[t]; }
        }
        ys[bl][j] = yv;
        us[bl][j] = uv;
    }
    if (threadIdx.x < JP) {
        ys[NARROW_SAMPLES][threadIdx.x] = -INFINITY;
        us[NARROW_SAMPLES][threadIdx.x] = 0.0f;
    }

    const bool is_input = i < I;
    const unsigned ic = (unsigned)min(i, I - 1);
    // the lane's input of every sample its wavefront takes, requested before anything waits
    constexpr int PER_WAVE = NARROW_SAMPLES / NARROW_WAVES;
    const float* __restrict__ xcol = x + (size_t)b0 * I + ic;
    float xs[PER_WAVE];
#pragma unroll
    for (int q = 0; q < PER_WAVE; ++q) {
        const int bl = min(wave + q * NARROW_WAVES, n_s - 1);
        xs[q] = is_input ? xcol[(size_t)bl * I] : biasvolt;
    }
    float wr[JL], acc[JL];
#pragma unroll
    for (int c = 0; c < JL; ++c) {
        wr[c] = (dx && is_input && j0 + c < J) ? w[(size_t)ic * J + j0 + c] : 0.0f;
        acc[c] = 0.0f;
    }
    __syncthreads();

    // four samples at a time, without branches, so that their LDS reads and lane exchanges overlap
    constexpr int BATCH = 4;
    static_assert(PER_WAVE % BATCH == 0, "samples per wavefront must be a multiple of the batch");
#pragma unroll
    for (int q0 = 0; q0 < PER_WAVE; q0 += BATCH) {
        float dxa[BATCH];
#pragma unroll
        for (int u = 0; u < BATCH; ++u) {
            const int bl = wave + (q0 + u) * NARROW_WAVES;
            const int row = bl < n_s ? bl : NARROW_SAMPLES;
            const float xq = xs[q0 + u] * -neg_s;
            dxa[u] = 0.0f;
#pragma unroll
            for (int c = 0; c < JL; ++c) {
                const float yv = ys[row][j0 + c], uv = us[row][j0 + c];
                acc[c] = __fmaf_rn(__builtin_amdgcn_fmed3f(yv - xq, 0.0f, 1.0f), uv, acc[c]);
                dxa[u] = __fmaf_rn(uv, xq <= yv ? wr[c] : 0.0f, dxa[u]);
            }
        }
        if (dx) {                                           // block-uniform
#pragma unroll
            for (int u = 0; u < BATCH; ++u) dxa[u] += __shfl_xor(dxa[u], NARROW_ROWS, kWave);      // (0 + 1), (2 + 3)
#pragma unroll
            for (int u = 0; u < BATCH; ++u) dxa[u] += __shfl_xor(dxa[u], 2 * NARROW_ROWS, kWave);
#pragma unroll
            for (int u = 0; u < BATCH; ++u) {
                const int bl = wave + (q0 + u) * NARROW_WAVES;
                if (group == 0 && is_input && bl < n_s) dx[(size_t)(b0 + bl) * I + i] = dxa[u];
            }
        }
    }

    if (!dst) return;
    if (wave > 0) {
#pragma unroll
        for (int c = 0; c < JL; ++c) red[wave - 1][c][lane] = acc[c];
    }
    __syncthreads();
    if (wave == 0 && i < rows) {
        float* out = dst + (size_t)blockIdx.y * rows * J + (size_t)i * J + j0;
#pragma unroll
        for (int c = 0; c < JL; ++c) {
            if (j0 + c < J) {
                float sum = acc[c];
#pragma unroll
                for (int v = 0; v < NARROW_WAVES - 1; ++v) sum += red[v][c][lane];
                out[c] = sum * post;
            }
        }
    }
}

// A block adds up 32 elements: its eight groups of 32 threads each take a contiguous eighth of the
// slices (two chains per thread keep loads in flight) and the eight sums are added in group order.
// The order of additions depends only on nsplit, never on timing.
constexpr int RED_ELEMS = 32, RED_GROUPS = 8;

__global__ void __launch_bounds__(RED_ELEMS * RED_GROUPS)
reduce_partials_kernel(const float* __restrict__ partial, float* __restrict__ out, int64_t n, int nsplit) {
    __shared__ float part[RED_GROUPS][RED_ELEMS];
    const int e = threadIdx.x % RED_ELEMS, g = threadIdx.x / RED_ELEMS;
    const int64_t t = (int64_t)blockIdx.x * RED_ELEMS + e;
    const int per = (nsplit + RED_GROUPS - 1) / RED_GROUPS;
    const int z_lo = g * per, z_hi = min(nsplit, z_lo + per);
    float a0 = 0.0f, a1 = 0.0f;
    if (t < n) {
        int z = z_lo;
        for (; z + 2 <= z_hi; z += 2) {
            a0 += partial[(size_t)z * n + t];
            a1 += partial[(size_t)(z + 1) * n + t];
        }
        if (z < z_hi) a0 += partial[(size_t)z * n + t];
    }
    part[g][e] = a0 + a1;
    __syncthreads();
    if (g == 0 && t < n) {
        float sum = part[0][e];
#pragma unroll
        for (int k = 1; k < RED_GROUPS; ++k) sum += part[k][e];
        out[t] = sum;
    }
}

// ---------------------------------------------------------------------------------------------
// Conv dX for layers the channel-lane kernel does not take (output channels not a multiple of 16, or fewer
// than 32 input channels under a kernel that is not three columns wide): the
// gradient per patch element, dxp[S, P], comes from the dense kernel above run over the implicit
// patches; here every element of the padded image adds up the patch elements that alias it, in
// (kh, kw) order.  Gather form: no atomics, fixed summation order.
// ---------------------------------------------------------------------------------------------
__global__ void __launch_bounds__(256)
cv_col2im_kernel(const float* __restrict__ dxp, float* __restrict__ dx, CropGeom crop, int64_t n, int H, int W, int C,
                 int Kh, int Kw, int Sh, int Sw, int Nh, int Nw) {
    const int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (t >= n) return;
    const int c = (int)(t % C);
    const int64_t pix = t / C;
    const int wx = (int)(pix % W);
    const int64_t rowi = pix / W;
    const int h = (int)(rowi % H);
    const int a = (int)(rowi / H);
    const int oh = h - crop.top, ow = wx - crop.left;         // only the caller's window is stored
    if (oh < 0 || oh >= crop.h || ow < 0 || ow >= crop.w) return;
    const int P = Kh * Kw * C;
    float acc = 0.0f;
    for (int kh = 0; kh < Kh; ++kh) {
        const int hh = h - kh;
        if (hh < 0 || hh % Sh != 0 || hh / Sh >= Nh) continue;
        for (int kw = 0; kw < Kw; ++kw) {
            const int ww = wx - kw;
            if (ww < 0 || ww % Sw != 0 || ww / Sw >= Nw) continue;
            const size_t s = (size_t)(a * Nh + hh / Sh) * Nw + ww / Sw;
            acc += dxp[s * P + (kh * Kw + kw) * C + c];
        }
    }
    dx[(((size_t)a * crop.h + oh) * crop.w + ow) * C + c] = acc;
}

int blocks_for(int64_t n, int block) { return (int)((n + block - 1) / block); }

}  // namespace

int launch_backward_prologue(const float* grad, const float* y, const float* rcp, float* upm, int64_t n,
                             const NeuronParams& np, int mode, const float* w, float* wt, int64_t rows,
                             int64_t cols, int64_t chan, float* zeros, int n_zeros, hipStream_t stream) {
    if (!zeros) n_zeros = 0;
    const bool vec4 = n % 4 == 0 && (((uintptr_t)grad | (uintptr_t)y | (uintptr_t)rcp | (uintptr_t)upm) & 15) == 0;
    const int64_t prep_blocks = vec4 ? (n / 4 + 255) / 256 : (n + 255) / 256;
    int64_t copy_blocks = 0;
    if (mode == 1) copy_blocks = ((cols + 31) / 32) * ((rows + 31) / 32);
    else if (mode == 2) copy_blocks = (rows * (cols / 4) + 255) / 256;
    if (mode != 0 && (rows <= 0 || cols <= 0)) { mode = 0; copy_blocks = 0; }
    if (prep_blocks + copy_blocks <= 0) return n_zeros > 0 ? launch_fill_zero(zeros, n_zeros, stream) : SNNTC_OK;
    if (prep_blocks + copy_blocks > 0x7fffffffLL) return fail(SNNTC_ERR_TOO_LARGE, "backward: grid too large");
    {
        KernelTimerScope timer_("prep_upstream", stream);
        hipLaunchKernelGGL(backward_prologue_kernel, dim3((unsigned)(prep_blocks + copy_blocks)), dim3(256), 0, stream,
                           grad, y, rcp, upm, n, np.max_cmp, (int)prep_blocks, vec4 ? 1 : 0, mode, w, wt, (int)rows, (int)cols,
                           (int)chan, zeros, n_zeros);
    }
    SNNTC_HIP_CHECK(hipGetLastError());
    return SNNTC_OK;
}

int launch_fill_zero(float* p, int64_t n, hipStream_t stream) {
    if (n <= 0) return SNNTC_OK;
    { KernelTimerScope timer_("fill_zero", stream);
    hipLaunchKernelGGL(fill_zero_kernel, dim3(blocks_for(n, 256)), dim3(256), 0, stream, p, n);
    }
    SNNTC_HIP_CHECK(hipGetLastError());
    return SNNTC_OK;
}

int launch_fc_grad_input(const float* x, const float* wt, const float* upm, const float* ym, float* dx,
                         int64_t B, int64_t I, int64_t J, int64_t wt_stride, hipStream_t stream) {
    if (B <= 0 || I <= 0) return SNNTC_OK;
    if (J <= 0) return launch_fill_zero(dx, B * I, stream);
    dim3 grid((unsigned)((B + DX_RB - 1) / DX_RB), (unsigned)((I + kWave - 1) / kWave));
    if (grid.y > 65535u) return fail(SNNTC_ERR_TOO_LARGE, "dense backward: input size %lld too large", (long long)I);
    { KernelTimerScope timer_("fc_grad_input", stream);
    SegmentSource src{};
    src.base = x; src.conv = 0; src.I = (int)I;
    hipLaunchKernelGGL(fc_grad_input_kernel<false>, grid, dim3(256), 0, stream, src, wt, upm, ym, dx, (int)B, (int)I,
                       (int)J, (int)wt_stride);
    }
    SNNTC_HIP_CHECK(hipGetLastError());
    return SNNTC_OK;
}

// Number of slices the segment range is cut into for dW: none when the (row-block x column-block)
// grid alone fills the chip; otherwise up to ~1536 blocks (six per CU, all resident at once), at
// least 64 segments per slice, at most 256 slices.  Within the upper half of that range the count
// is the one whose blocks spread most evenly over the 256 CUs: the launch lasts as long as the CU
// with the most blocks, ceil(blocks / 256) of them, each 1/n of a column of work.
int weight_grad_splits(int64_t S, int64_t base_blocks) {
    if (base_blocks >= 1024) return 1;
    if (base_blocks < 1) base_blocks = 1;
    int64_t want = (1536 + base_blocks - 1) / base_blocks;
    int64_t cap = S / 64;
    if (want > cap) want = cap;
    if (want > 256) want = 256;
    if (want < 1) want = 1;
    int64_t best = want;
    double best_cost = 1e30;
    for (int64_t n = want; n >= 1 && 2 * n >= want; --n) {
        const double cost = (double)((base_blocks * n + 255) / 256) / (double)n;
        if (cost < best_cost * 0.995) { best_cost = cost; best = n; }
    }
    return (int)best;
}

int grad_weight_blocks(int64_t rows, int64_t J) {
    return (int)(((J + kWave - 1) / kWave) * ((rows + DW_RI - 1) / DW_RI));
}

// Rows [row_start, rows) of dW, or of every partial-sum slice when nsplit > 1 (dst = slices).
int launch_grad_weight_rows(const SegmentSource& src, const float* upm, const float* ym, float* dst,
                            int nsplit, int64_t S, int64_t J, int64_t row_start, const NeuronParams& np,
                            hipStream_t stream) {
    const int64_t rows = (int64_t)src.I + np.bias;
    if (rows <= row_start || J <= 0 || S <= 0) return SNNTC_OK;
    if (nsplit < 1) nsplit = 1;
    const int seg_per_slice = (int)((S + nsplit - 1) / nsplit);
    dim3 grid((unsigned)((J + kWave - 1) / kWave), (unsigned)((rows - row_start + DW_RI - 1) / DW_RI),
              (unsigned)nsplit);
    if (grid.y > 65535u) return fail(SNNTC_ERR_TOO_LARGE, "weight gradient: too many weight rows");
    {
        KernelTimerScope timer_(row_start ? "grad_weight_tail" : "grad_weight", stream);
        const LeadScale ls = lead_scale(np.max_time);
        // (the dense kernel addresses a slice of ym / upm with 32-bit byte offsets)
        if (!src.conv && row_start == 0 && ((int64_t)seg_per_slice + DWD_TILE) * J * (int64_t)sizeof(float) < 0x7fffffffLL)
            hipLaunchKernelGGL(grad_weight_dense_kernel, grid, dim3(256), 0, stream, src.base, upm, ym, dst, (int)S,
                               (int)src.I, (int)J, (int)rows, seg_per_slice, np.biasvolt, ls.neg_s, ls.post);
        else
            hipLaunchKernelGGL(grad_weight_kernel, grid, dim3(256), 0, stream, src, upm, ym, dst, (int)S, (int)J,
                               (int)rows, (int)row_start, seg_per_slice, np.biasvolt, ls.neg_s, ls.post);
    }
    SNNTC_HIP_CHECK(hipGetLastError());
    return SNNTC_OK;
}

int launch_reduce_partials(const float* partial, float* dw, int64_t n, int nsplit, hipStream_t stream) {
    if (n <= 0 || nsplit <= 1) return SNNTC_OK;
    {
        KernelTimerScope timer_("reduce_partials", stream);
        hipLaunchKernelGGL(reduce_partials_kernel, dim3(blocks_for(n, RED_ELEMS)), dim3(RED_ELEMS * RED_GROUPS), 0,
                           stream, partial, dw, n, nsplit);
    }
    SNNTC_HIP_CHECK(hipGetLastError());
    return SNNTC_OK;
}

bool fc_backward_narrow_supported(int64_t J) { return J >= 1 && J <= NARROW_JMAX; }

int fc_backward_narrow_splits(int64_t B) { return (int)((B + NARROW_SAMPLES - 1) / NARROW_SAMPLES); }

// dx and/or dw may be NULL.  With more than one block of samples `partial` takes the dW slices.
int launch_fc_backward_narrow(const float* x, const float* w, const float* grad, const float* y, const float* rcp,
                              float* dx, float* dw, float* partial, float* zeros, int n_zeros, int64_t B, int64_t I,
                              int64_t J, const NeuronParams& np, hipStream_t stream) {
    if (!zeros) n_zeros = 0;
    const int64_t rows = I + np.bias;
    const int nsplit = fc_backward_narrow_splits(B);
    // without dW only the input rows are needed; the bias row has no dX
    const int64_t lanes = dw ? rows : I;
    dim3 grid((unsigned)((lanes + NARROW_ROWS - 1) / NARROW_ROWS), (unsigned)nsplit);
    if (grid.y > 65535u) return fail(SNNTC_ERR_TOO_LARGE, "dense backward: batch %lld too large", (long long)B);
    float* dst = dw ? (nsplit > 1 ? partial : dw) : nullptr;
    {
        KernelTimerScope timer_("fc_backward_narrow", stream);
        const LeadScale ls = lead_scale(np.max_time);
        const int jl = (int)((J + NARROW_GROUPS - 1) / NARROW_GROUPS);      // columns per lane
        auto kern = jl == 1 ? fc_backward_narrow_kernel<1> : jl == 2 ? fc_backward_narrow_kernel<2>
                  : jl == 3 ? fc_backward_narrow_kernel<3> : fc_backward_narrow_kernel<4>;
        hipLaunchKernelGGL(kern, grid, dim3(NARROW_WAVES * kWave), 0, stream, x, w, grad, y, rcp, dx, dst, (int)B,
                           (int)I, (int)J, (int)rows, np.max_cmp, np.biasvolt, ls.neg_s, ls.post, zeros, n_zeros);
    }
    SNNTC_HIP_CHECK(hipGetLastError());
    if (!dw) return SNNTC_OK;
    return launch_reduce_partials(partial, dw, rows * J, nsplit, stream);
}

// dxp: scratch of S * P floats (gradient per patch element)
int launch_cv_grad_input(const SegmentSource& src, const float* wt, const float* upm, const float* ym, float* dxp,
                         float* dx, const CropGeom& crop, const ConvGeom& g, int64_t wt_stride, hipStream_t stream) {
    const int64_t n = g.B * g.H * g.W * g.C;
    if (n <= 0) return SNNTC_OK;
    if (g.Kc <= 0 || g.S <= 0) return launch_fill_zero(dx, g.B * crop.h * crop.w * g.C, stream);
    dim3 grid((unsigned)((g.S + DX_RB - 1) / DX_RB), (unsigned)((g.P + kWave - 1) / kWave));
    if (grid.y > 65535u) return fail(SNNTC_ERR_TOO_LARGE, "conv backward: patch length %lld too large", (long long)g.P);
    { KernelTimerScope timer_("cv_grad_input", stream);
    hipLaunchKernelGGL(fc_grad_input_kernel<true>, grid, dim3(256), 0, stream, src, wt, upm, ym, dxp, (int)g.S,
                       (int)g.P, (int)g.Kc, (int)wt_stride);
    }
    SNNTC_HIP_CHECK(hipGetLastError());
    { KernelTimerScope timer_("cv_col2im", stream);
    hipLaunchKernelGGL(cv_col2im_kernel, dim3(blocks_for(n, 256)), dim3(256), 0, stream, dxp, dx, crop, n, (int)g.H,
                       (int)g.W, (int)g.C, (int)g.Kh, (int)g.Kw, (int)g.Sh, (int)g.Sw, (int)g.Nh, (int)g.Nw);
    }
    SNNTC_HIP_CHECK(hipGetLastError());
    return SNNTC_OK;
}

}  // namespace snntc
