// Causal-set scan: for every (segment, output neuron) walk the segment's inputs in ascending
// order, accumulate sum(w) and sum(w*z), and stop at the first prefix whose weighted mean lies
// after its last input and not after the next one.
//
// Replaces SnnFcCudaOutKernel / SnnFcCudaOutKernelBias (snntc/snnfc_kernels.cu.cc:19-71,
// snntc/snncv_kernels.cu.cc:19-72) and reproduces their arithmetic step by step: bias first,
// sequential fp32 accumulation with a fused multiply-add for ysum, the division-free firing test
// |ysum| > x*|wsum| with the product rounded on its own, and y = ysum * (1/wsum).
//
// Kernels, by launch size (launch_scan_lds picks):
//   scan_filter_kernel     large and mid-sized launches: weight slice in LDS, one or two neurons per
//                          lane, and the tests of a step skipped wherever a margin test on a whole
//                          chunk of eight inputs proves that none of them can close the set;
//   scan_lds_kernel        small launches (a couple of wavefronts per SIMD): weight slice in LDS, every
//                          step with its tests, written for latency;
//   scan_lds_split_kernel  fewer work items than CUs: one item per workgroup, its weights gathered
//                          into LDS in scan order first, then one wavefront accumulating and the
//                          others sharing the item's tests;
//   scan_kernel            segments so long that not even eight weight columns fit in LDS: weight
//                          rows streamed from memory, one wavefront per (segment, 64 neurons).
// In all of them lanes run across neurons, so a weight row is read coalesced (or conflict-free from
// LDS), while the sorted value and the row index of a step are the same for all lanes of a segment
// (segment rows are padded to a multiple of 16 entries so that they are fetched eight at a time
// without bounds checks).
#include <atomic>
#include <type_traits>
#include <utility>

#include "snntc_common.h"

namespace snntc {
namespace {

constexpr int CHUNK = 8;

struct LaneState {
    float wsum, ysum, wa, ya;
    bool fired;
};

// One scan step for a lane that is still open.  Returns false when the causal set closes before
// consuming input x (the lane then keeps its state).
__device__ __forceinline__ bool scan_step(LaneState& s, float x, float wv) {
    if (s.fired && s.ya <= x * s.wa) return false;
    s.wsum += wv;
    s.ysum = __fmaf_rn(x, wv, s.ysum);
    s.wa = fabsf(s.wsum);
    s.ya = s.wsum < 0.0f ? -s.ysum : s.ysum;
    s.fired = s.ya > x * s.wa;
    return true;
}

template <bool WANT_K>
__global__ void __launch_bounds__(256)
scan_kernel(const float* __restrict__ sorted, const int32_t* __restrict__ perm,
            const int32_t* __restrict__ n_real, const float* __restrict__ w, float* __restrict__ y_out,
            float* __restrict__ rcp_out, int32_t* __restrict__ k_out, int64_t n_items, int I, int stride,
            int J, int j_blocks, NeuronParams np, TimeCopy copy) {
    // work item = (segment, 64-neuron block); one per wavefront
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
    const int64_t item = (int64_t)blockIdx.x * (blockDim.x / kWave) + wave;
    if (item >= n_items) return;
    const int seg = (int)(item / j_blocks);
    const int jb = (int)(item - (int64_t)seg * j_blocks);
    const int lane = threadIdx.x % kWave;
    const int j = jb * kWave + lane;
    const bool active = j < J;
    const unsigned jc = (unsigned)(active ? j : J - 1);      // clamp so every lane reads valid memory

    const float* __restrict__ xs = sorted + (size_t)seg * stride;
    const int32_t* __restrict__ pr = perm + (size_t)seg * stride;
    const int n = n_real[seg];                                // inputs with value <= MAX-0.1

    LaneState s;
    s.wsum = -np.theta; s.ysum = 0.0f; s.wa = 0.0f; s.ya = 0.0f; s.fired = false;
    if (np.bias) {
        const float wb = (w + (size_t)I * J)[jc];
        s.wsum += wb;
        s.ysum = np.biasvolt * wb;
        s.wa = fabsf(s.wsum);
        s.ya = s.wsum < 0.0f ? -s.ysum : s.ysum;
        s.fired = s.ya > s.wa * np.biasvolt;
    }

    int kcnt = 0;
    if (active) {
        // w[row, j]: the row base is wave-uniform (scalar registers), the lane adds a 32-bit byte offset
        const unsigned joff = jc * (unsigned)sizeof(float);
        auto weight_at = [&](int32_t row) -> float {
            const char* rowp = reinterpret_cast<const char*>(w + (uint32_t)row * (uint32_t)J);
            return *reinterpret_cast<const float*>(rowp + joff);
        };

        const int n_full = n & ~(CHUNK - 1);
        float wq[CHUNK];
#pragma unroll
        for (int u = 0; u < CHUNK; ++u) wq[u] = weight_at(pr[u]);    // row padding keeps pr[0..15] readable
        bool open = true;
        for (int k0 = 0; k0 < n_full && open; k0 += CHUNK) {
            float xv[CHUNK], wc[CHUNK];
            const int kn = (k0 + CHUNK < n_full) ? k0 + CHUNK : k0;  // next chunk, or a harmless re-read
#pragma unroll
            for (int u = 0; u < CHUNK; ++u) {
                xv[u] = xs[k0 + u];
                wc[u] = wq[u];
                wq[u] = weight_at(pr[kn + u]);
            }
#pragma unroll
            for (int u = 0; u < CHUNK; ++u) {
                if (open) {
                    open = scan_step(s, xv[u], wc[u]);
                    if (WANT_K && open) kcnt = k0 + u + 1;
                }
            }
        }
        // up to CHUNK-1 trailing steps
        for (int k = n_full; k < n && open; ++k) {
            open = scan_step(s, xs[k], weight_at(pr[k]));
            if (WANT_K && open) kcnt = k + 1;
        }

        float y = np.max_time, r = 0.0f;
        if (s.fired) {
            r = 1.0f / s.wsum;
            y = s.ysum * r;
            if (y >= np.max_time) { y = np.max_time; r = 0.0f; }
        }
        const size_t o = (size_t)seg * J + j;
        y_out[o] = y;
        rcp_out[o] = r;
        if (copy.dst) copy.dst[time_copy_pixel(copy, seg) * J + j] = y;
        if (WANT_K) k_out[o] = (s.fired && r != 0.0f) ? kcnt : -1;
    }
}

// ---------------------------------------------------------------------------------------------
// Scan with the weight slice resident in LDS.
//
// Walking W rows in sorted order from memory re-reads the whole matrix once per segment (8 GB of
// cache traffic for 65 536 patches of a 3x3x64 -> 64 layer).  Here a workgroup copies the COLS
// columns it owns -- all I(+1) rows, at most 160 KB -- into LDS once and then scans many segments
// against it.  A wavefront covers 64/COLS segments at a time (lanes = segment x column), so narrow
// layers (J = 10, Kc = 32) and long segments (COLS = 8 for 4608 inputs) use the same kernel.
// Sorted values and row indices are fetched per lane (all lanes of a segment read the same
// address) eight steps at a time, one chunk ahead of the LDS reads that need them.
// ---------------------------------------------------------------------------------------------
constexpr int LDS_SCAN_THREADS = 1024;
constexpr int LDS_SCAN_BYTES = 160 * 1024;
// The widest slice that fits is taken: the register budget allows one 16-wave workgroup per CU anyway,
// and fewer slices re-read the sorted rows less often.
// Behind the slice: 64 bytes for a reduction and room for the chunk buffers of at least four
// wavefronts (scan_filter_kernel: 64 bytes per segment of a wavefront, at most 8 segments).
constexpr int FILTER_XBUF_SEG_BYTES = 2 * CHUNK * (int)sizeof(float);
constexpr int LDS_SCAN_TARGET = 160 * 1024 - 64 - 4 * 8 * FILTER_XBUF_SEG_BYTES;

struct Chunk {
    float x[CHUNK];
    int32_t p[CHUNK];
};

// Rows are read through buffer descriptors: a scalar descriptor (first row of the work item), a
// scalar chunk offset and a per-lane byte offset that never changes during a scan.  No per-lane
// address arithmetic is left, so issuing the next loads never has to wait for those in flight.
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));

struct RowSource {
    __amdgpu_buffer_rsrc_t xs, pr;
};

__device__ __forceinline__ RowSource make_row_source(const float* xs0, const int32_t* pr0, int bytes) {
    RowSource r;
    r.xs = __builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(xs0), 0, bytes, 0x00020000);
    r.pr = __builtin_amdgcn_make_buffer_rsrc(const_cast<int32_t*>(pr0), 0, bytes, 0x00020000);
    return r;
}

__device__ __forceinline__ void load_chunk_flat(Chunk& c, const float* __restrict__ xs,
                                                const int32_t* __restrict__ pr, int k) {
    const float4 a = *reinterpret_cast<const float4*>(xs + k);
    const float4 b = *reinterpret_cast<const float4*>(xs + k + 4);
    const int4 pa = *reinterpret_cast<const int4*>(pr + k);
    const int4 pb = *reinterpret_cast<const int4*>(pr + k + 4);
    c.x[0] = a.x; c.x[1] = a.y; c.x[2] = a.z; c.x[3] = a.w;
    c.x[4] = b.x; c.x[5] = b.y; c.x[6] = b.z; c.x[7] = b.w;
    c.p[0] = pa.x; c.p[1] = pa.y; c.p[2] = pa.z; c.p[3] = pa.w;
    c.p[4] = pb.x; c.p[5] = pb.y; c.p[6] = pb.z; c.p[7] = pb.w;
}

__device__ __forceinline__ void load_chunk(Chunk& c, const RowSource& src, int lane_bytes, int k) {
    const u32x4 a = __builtin_amdgcn_raw_buffer_load_b128(src.xs, lane_bytes, k * 4, 0);
    const u32x4 b = __builtin_amdgcn_raw_buffer_load_b128(src.xs, lane_bytes + 16, k * 4, 0);
    const u32x4 pa = __builtin_amdgcn_raw_buffer_load_b128(src.pr, lane_bytes, k * 4, 0);
    const u32x4 pb = __builtin_amdgcn_raw_buffer_load_b128(src.pr, lane_bytes + 16, k * 4, 0);
    c.x[0] = __uint_as_float(a.x); c.x[1] = __uint_as_float(a.y); c.x[2] = __uint_as_float(a.z);
    c.x[3] = __uint_as_float(a.w); c.x[4] = __uint_as_float(b.x); c.x[5] = __uint_as_float(b.y);
    c.x[6] = __uint_as_float(b.z); c.x[7] = __uint_as_float(b.w);
    c.p[0] = (int)pa.x; c.p[1] = (int)pa.y; c.p[2] = (int)pa.z; c.p[3] = (int)pa.w;
    c.p[4] = (int)pb.x; c.p[5] = (int)pb.y; c.p[6] = (int)pb.z; c.p[7] = (int)pb.w;
}

#define SNNTC_SCAN_COUNT "v_add_u32_e32 %[kcnt], 1, %[kcnt]\n"
#define SNNTC_SCAN_INPUTS(XC, X)                                                                       \
    [run] "s"(run), [x0] XC(X[0]), [x1] XC(X[1]), [x2] XC(X[2]), [x3] XC(X[3]), [x4] XC(X[4]),          \
        [x5] XC(X[5]), [x6] XC(X[6]), [x7] XC(X[7]), [w0] "v"(w[0]), [w1] "v"(w[1]), [w2] "v"(w[2]),    \
        [w3] "v"(w[3]), [w4] "v"(w[4]), [w5] "v"(w[5]), [w6] "v"(w[6]), [w7] "v"(w[7])

// Eight scan steps for the lanes in `run`, written out by hand, every decision on the vector side:
// the lane carries a gate value yg = fired ? ya : +inf, the closing test `yg > x*|wsum|` writes
// EXEC directly (a lane that closes drops out of the rest of the block) and the new gate is a
// select.  Per step (x = input time, w = its weight), nine vector instructions and no branch:
//     EXEC &= yg > x*|wsum|                       (a closing lane keeps its sums)
//     wsum  += w ; ysum = fma(x, w, ysum) ; ya = wsum < 0 ? -ysum : ysum
//     yg     = ya > x*|wsum| ? ya : +inf
// No vector -> scalar -> EXEC round trips, so a step of a lone wavefront takes few cycles.
#define SNNTC_VSCAN_STEP(U)                                                  \
    "v_mul_f32_e64 %[t], %[x" #U "], |%[wsum]|\n"                            \
    "v_cmpx_gt_f32_e32 vcc, %[yg], %[t]\n"                                   \
    "v_add_f32_e32 %[wsum], %[wsum], %[w" #U "]\n"                           \
    "v_fmac_f32_e32 %[ysum], %[x" #U "], %[w" #U "]\n"                       \
    "v_cmp_gt_f32_e32 vcc, 0, %[wsum]\n"                                     \
    "v_cndmask_b32_e64 %[ya], %[ysum], -%[ysum], vcc\n"                      \
    "v_mul_f32_e64 %[t], %[x" #U "], |%[wsum]|\n"                            \
    "v_cmp_gt_f32_e32 vcc, %[ya], %[t]\n"                                    \
    "v_cndmask_b32_e32 %[yg], %[inf], %[ya], vcc\n"
#define SNNTC_VSCAN_PROLOGUE                        \
    "s_mov_b64 %[save], exec\n"                     \
    "s_mov_b64 exec, %[run]\n"
#define SNNTC_VSCAN_EPILOGUE                         \
    "s_andn2_b64 %[gone], %[run], exec\n"            \
    "s_or_b64 %[closed], %[closed], %[gone]\n"       \
    "s_mov_b64 exec, %[save]\n"
#define SNNTC_VSCAN_STATE                                                                              \
    [wsum] "+v"(wsum), [ysum] "+v"(ysum), [ya] "+v"(ya), [yg] "+v"(yg), [kcnt] "+v"(kcnt),             \
        [closed] "+s"(closed), [save] "=&s"(saved_exec), [gone] "=&s"(gone), [t] "=&v"(t)
#define SNNTC_VSCAN_INPUTS                                                                             \
    [run] "s"(run), [inf] "v"(inf), [x0] "v"(x[0]), [x1] "v"(x[1]), [x2] "v"(x[2]), [x3] "v"(x[3]),     \
        [x4] "v"(x[4]), [x5] "v"(x[5]), [x6] "v"(x[6]), [x7] "v"(x[7]), [w0] "v"(w[0]), [w1] "v"(w[1]), \
        [w2] "v"(w[2]), [w3] "v"(w[3]), [w4] "v"(w[4]), [w5] "v"(w[5]), [w6] "v"(w[6]), [w7] "v"(w[7])

template <bool WANT_K>
__device__ __forceinline__ void scan_chunk_vector(float& wsum, float& ysum, float& ya, float& yg, int& kcnt,
                                                  uint64_t& closed, uint64_t run, const float (&x)[CHUNK],
                                                  const float (&w)[CHUNK]) {
    uint64_t saved_exec, gone;
    float t;
    const float inf = INFINITY;
    if (WANT_K)
        asm volatile(SNNTC_VSCAN_PROLOGUE SNNTC_VSCAN_STEP(0) SNNTC_SCAN_COUNT SNNTC_VSCAN_STEP(1) SNNTC_SCAN_COUNT
                     SNNTC_VSCAN_STEP(2) SNNTC_SCAN_COUNT SNNTC_VSCAN_STEP(3) SNNTC_SCAN_COUNT SNNTC_VSCAN_STEP(4)
                     SNNTC_SCAN_COUNT SNNTC_VSCAN_STEP(5) SNNTC_SCAN_COUNT SNNTC_VSCAN_STEP(6) SNNTC_SCAN_COUNT
                     SNNTC_VSCAN_STEP(7) SNNTC_SCAN_COUNT SNNTC_VSCAN_EPILOGUE
                     : SNNTC_VSCAN_STATE : SNNTC_VSCAN_INPUTS : "vcc", "scc");
    else
        asm volatile(SNNTC_VSCAN_PROLOGUE SNNTC_VSCAN_STEP(0) SNNTC_VSCAN_STEP(1) SNNTC_VSCAN_STEP(2)
                     SNNTC_VSCAN_STEP(3) SNNTC_VSCAN_STEP(4) SNNTC_VSCAN_STEP(5) SNNTC_VSCAN_STEP(6)
                     SNNTC_VSCAN_STEP(7) SNNTC_VSCAN_EPILOGUE
                     : SNNTC_VSCAN_STATE : SNNTC_VSCAN_INPUTS : "vcc", "scc");
}

// Eight inputs added to the running sums of the lanes in `run`, no tests: what a wavefront does for
// the chunks whose tests another wavefront of its workgroup evaluates (scan_lds_split_kernel).
#define SNNTC_ACC_STEP(U)                                  \
    "v_add_f32_e32 %[wsum], %[wsum], %[w" #U "]\n"         \
    "v_fmac_f32_e32 %[ysum], %[x" #U "], %[w" #U "]\n"
__device__ __forceinline__ void accumulate_chunk(float& wsum, float& ysum, int& kcnt, uint64_t run,
                                                 const float (&x)[CHUNK], const float (&w)[CHUNK]) {
    uint64_t saved_exec;
    asm volatile("s_mov_b64 %[save], exec\n"
                 "s_mov_b64 exec, %[run]\n" SNNTC_ACC_STEP(0) SNNTC_ACC_STEP(1) SNNTC_ACC_STEP(2) SNNTC_ACC_STEP(3)
                     SNNTC_ACC_STEP(4) SNNTC_ACC_STEP(5) SNNTC_ACC_STEP(6) SNNTC_ACC_STEP(7)
                 "v_add_u32_e32 %[kcnt], 8, %[kcnt]\n"
                 "s_mov_b64 exec, %[save]\n"
                 : [wsum] "+v"(wsum), [ysum] "+v"(ysum), [kcnt] "+v"(kcnt), [save] "=&s"(saved_exec)
                 : SNNTC_SCAN_INPUTS("v", x));
}

// Copies columns [j0, j0 + COLS) of all `rows` rows of W[rows, J] into LDS as wl[row][COLS] (zeros
// past column J).  Loads are issued in batches so that a small workgroup does not pay one memory
// latency per element.
// Returns the largest |w| among the values this thread copied (NaN entries skipped).
template <int COLS>
__device__ __forceinline__ float fill_weight_slice(float* __restrict__ wl, const float* __restrict__ w, int rows,
                                                   int J, int j0) {
    const int n_fill = rows * COLS;
    float amax = 0.0f;
    if ((J & 3) == 0) {
        constexpr int C4 = COLS / 4, FILL = 4;
        for (int base = threadIdx.x; base < rows * C4; base += FILL * blockDim.x) {
            float4 v[FILL];
#pragma unroll
            for (int u = 0; u < FILL; ++u) {
                const int idx = base + u * blockDim.x;
                const int r = idx / C4, c = (idx - r * C4) * 4;
                v[u] = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
                if (idx < rows * C4 && j0 + c < J) v[u] = *reinterpret_cast<const float4*>(w + (size_t)r * J + j0 + c);
            }
#pragma unroll
            for (int u = 0; u < FILL; ++u) {
                const int idx = base + u * blockDim.x;
                if (idx < rows * C4) reinterpret_cast<float4*>(wl)[idx] = v[u];
                amax = fmaxf(amax, fmaxf(fmaxf(fabsf(v[u].x), fabsf(v[u].y)), fmaxf(fabsf(v[u].z), fabsf(v[u].w))));
            }
        }
    } else if (j0 == 0 && J > 1 && J < COLS && (reinterpret_cast<uintptr_t>(w) & 15) == 0 && rows * J < (1 << 24)) {
        // One slice holds every column (a 10-wide head): the source is a single run of rows*J floats.
        // It is read as aligned float4 regardless of J, eight per thread in flight, and each value
        // is dropped at [row][col]; the padding columns are zeroed first.
        for (int idx = threadIdx.x; idx < n_fill / 4; idx += blockDim.x)
            reinterpret_cast<float4*>(wl)[idx] = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
        __syncthreads();
        constexpr int FILL = 8;
        const int n = rows * J, n4 = n / 4;
        const unsigned magic = 0xffffffffu / (unsigned)J + 1;      // e / J == umulhi(e, magic) for e < 2^24
        for (int base = threadIdx.x; base < n4; base += FILL * blockDim.x) {
            float4 v[FILL];
#pragma unroll
            for (int u = 0; u < FILL; ++u) {
                const int idx = base + u * blockDim.x;
                if (idx < n4) v[u] = reinterpret_cast<const float4*>(w)[idx];
            }
#pragma unroll
            for (int u = 0; u < FILL; ++u) {
                const int idx = base + u * blockDim.x;
                if (idx < n4) {
                    const float q[4] = {v[u].x, v[u].y, v[u].z, v[u].w};
#pragma unroll
                    for (int t = 0; t < 4; ++t) {
                        const unsigned e = 4u * idx + t, r = __umulhi(e, magic);
                        wl[r * COLS + (e - r * J)] = q[t];
                        amax = fmaxf(amax, fabsf(q[t]));
                    }
                }
            }
        }
        if ((int)threadIdx.x < n - 4 * n4) {
            const unsigned e = 4u * n4 + threadIdx.x, r = __umulhi(e, magic);
            const float v = w[e];
            wl[r * COLS + (e - r * J)] = v;
            amax = fmaxf(amax, fabsf(v));
        }
    } else {
        constexpr int FILL = 16;
        for (int base = threadIdx.x; base < n_fill; base += FILL * blockDim.x) {
            float v[FILL];
#pragma unroll
            for (int u = 0; u < FILL; ++u) {
                const int idx = base + u * blockDim.x;
                const int r = idx / COLS, c = idx - r * COLS;
                v[u] = (idx < n_fill && j0 + c < J) ? w[(size_t)r * J + j0 + c] : 0.0f;
            }
#pragma unroll
            for (int u = 0; u < FILL; ++u) {
                const int idx = base + u * blockDim.x;
                if (idx < n_fill) wl[idx] = v[u];
                amax = fmaxf(amax, fabsf(v[u]));
            }
        }
    }
    return amax;
}

// Launches with at most a couple of wavefronts per SIMD, where nothing hides a stall: workgroups of
// at most four wavefronts (so that the work spreads over the chip), one neuron per lane, seven chunks
// of (x, row) in flight through buffer loads, and the step-by-step block for every chunk (the
// filtered kernel below pays a fixed price per work item that such small launches do not win back).
constexpr int LOW_LATENCY_THREADS = 256;

template <int COLS, bool WANT_K>
__global__ void __launch_bounds__(LOW_LATENCY_THREADS)
scan_lds_kernel(const float* __restrict__ sorted, const int32_t* __restrict__ perm,
                const int32_t* __restrict__ n_real, const float* __restrict__ w, float* __restrict__ y_out,
                float* __restrict__ rcp_out, int32_t* __restrict__ k_out, int S, int I, int stride, int J,
                int n_slices, int n_groups, NeuronParams np, TimeCopy copy) {
    extern __shared__ __align__(16) float wl[];                          // [I + bias][COLS]
    constexpr int SEGS = kWave / COLS;                     // segments per wavefront
    const int WAVES = blockDim.x / kWave;                  // 1..4, chosen by the launcher
    // slice-major over XCD-contiguous ids: the workgroups of one XCD share a few weight slices
    const int block = xcd_contiguous(blockIdx.x, gridDim.x);
    const int slice = block / n_groups;
    const int group = block - slice * n_groups;
    const int j0 = slice * COLS;
    const int rows = I + np.bias;

    fill_weight_slice<COLS>(wl, w, rows, J, j0);
    __syncthreads();

    const int lane = threadIdx.x % kWave;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
    const int sub = lane / COLS, col = lane - sub * COLS;
    const int j = j0 + col;
    const float* __restrict__ wcol = wl + col;
    const int last_chunk = stride - CHUNK;                 // start of the last readable chunk of a row

    for (int item = group * WAVES + wave; item * SEGS < S; item += n_groups * WAVES) {
        const int seg_raw = item * SEGS + sub;
        const bool live = seg_raw < S && j < J;
        const int seg = seg_raw < S ? seg_raw : S - 1;      // idle lanes shadow a valid segment
        const float* __restrict__ xs = sorted + (size_t)seg * stride;
        const int32_t* __restrict__ pr = perm + (size_t)seg * stride;
        const int seg0 = __builtin_amdgcn_readfirstlane(item * SEGS);
        const int n_segs = S - seg0 < SEGS ? S - seg0 : SEGS;
        const RowSource rows_of_item = make_row_source(sorted + (size_t)seg0 * stride, perm + (size_t)seg0 * stride,
                                                       n_segs * stride * (int)sizeof(float));
        const int lane_bytes = (seg - seg0) * stride * (int)sizeof(float);
        const int n = live ? n_real[seg] : 0;
        const int n_full = n & ~(CHUNK - 1);

        float wsum = -np.theta, ysum = 0.0f, ya = 0.0f;
        bool fired0 = false;
        if (np.bias) {
            const float wb = wcol[I * COLS];
            wsum += wb;
            ysum = np.biasvolt * wb;
            ya = wsum < 0.0f ? -ysum : ysum;
            fired0 = ya > fabsf(wsum) * np.biasvolt;
        }
        uint64_t closed = 0;
        int kcnt = 0;
        float yg = fired0 ? ya : INFINITY;                  // gate value of the step block

        // NBUF chunks of (x, row) are held: c is consumed, c+1 feeds the LDS reads, up to c+NBUF-1
        // are being fetched.  The phase loop is unrolled so that buffer indices are compile-time.
        constexpr int NBUF = 8, AHEAD = NBUF - 1;
        Chunk xp[NBUF];
        float wv[2][CHUNK];
#pragma unroll
        for (int b = 0; b < AHEAD; ++b) load_chunk(xp[b], rows_of_item, lane_bytes, b * CHUNK <= last_chunk ? b * CHUNK : 0);
#pragma unroll
        for (int u = 0; u < CHUNK; ++u) wv[0][u] = wcol[xp[0].p[u] * COLS];

        // The body is one straight block per NBUF chunks (no exit between phases: a phase whose lanes
        // are all done runs with an empty EXEC), which lets the compiler keep all seven chunks in flight.
        for (int k0 = 0;; k0 += NBUF * CHUNK) {
#pragma unroll
            for (int ph = 0; ph < NBUF; ++ph) {
                __builtin_amdgcn_sched_barrier(0);          // keep each phase's loads and reads in it
                const int k = k0 + ph * CHUNK;
                const uint64_t run = __ballot(k < n_full) & ~closed;
                const int kn = k + AHEAD * CHUNK;
                load_chunk(xp[(ph + AHEAD) % NBUF], rows_of_item, lane_bytes, kn <= last_chunk ? kn : 0);
#pragma unroll
                for (int u = 0; u < CHUNK; ++u) wv[(ph + 1) % 2][u] = wcol[xp[(ph + 1) % NBUF].p[u] * COLS];
                scan_chunk_vector<WANT_K>(wsum, ysum, ya, yg, kcnt, closed, run, xp[ph % NBUF].x, wv[ph % 2]);
            }
            if ((__ballot(k0 + NBUF * CHUNK < n_full) & ~closed) == 0) break;
        }

        // per-lane epilogue: up to CHUNK-1 trailing inputs, then the output
        if (live) {
            LaneState s;
            s.wsum = wsum; s.ysum = ysum; s.wa = fabsf(wsum); s.ya = ya;
            const bool was_closed = (closed >> lane) & 1;
            s.fired = was_closed || yg < INFINITY;
            bool open = !was_closed;
            for (int k = n_full; k < n && open; ++k) {
                open = scan_step(s, xs[k], wcol[pr[k] * COLS]);
                if (WANT_K && open) ++kcnt;
            }
            float y = np.max_time, r = 0.0f;
            if (s.fired) {
                r = 1.0f / s.wsum;
                y = s.ysum * r;
                if (y >= np.max_time) { y = np.max_time; r = 0.0f; }
            }
            const size_t o = (size_t)seg * J + j;
            y_out[o] = y;
            rcp_out[o] = r;
            if (copy.dst) copy.dst[time_copy_pixel(copy, seg) * J + j] = y;
            if (WANT_K) k_out[o] = (s.fired && r != 0.0f) ? kcnt : -1;
        }
    }
}

// Launches of a few dozen work items (the 10-wide head of a classifier): one item per workgroup,
// its wavefronts sharing the item instead of taking one each.  The running sums of a scan are
// inherently sequential, its tests are not, and a lone wavefront pays about five clocks for every
// instruction it issues, whatever the instruction.  So the sequential part is stripped to the two
// additions per input and the reads that feed them:
//   * before the scan all wavefronts gather the item's weights in scan order, w[lane][k] =
//     W[perm[seg][k]][j], straight from memory into LDS (every entry is independent), next to the
//     sorted rows; the scans then read times and weights as 16-byte runs with no address
//     arithmetic, and the row indices never enter LDS;
//   * wavefront 0 (the producer) only accumulates; after every chunk of eight inputs it leaves
//     the sums in LDS and advances a progress counter.  While every scan of the item still has a
//     full round of four chunks ahead no lane is masked and nothing is compared;
//   * the other wavefronts (the testers) take every SPLIT_TESTERS-th chunk: they wait for the sums before their chunk,
//     recompute the fired state from them and the last input before the chunk, and run the ordinary
//     eight-step block with all its tests.  Each tester records the first close it sees; the
//     earliest of all is the scan's (a close found in a chunk is exact as long as no earlier step
//     closed, and an earlier close wins the minimum anyway).  The producer walks the trailing
//     inputs (fewer than eight) and supplies the result of a scan that never closes.
// An item is SPLIT lanes wide: 32 lanes (the upper half of the wavefronts mirrors the lower) keep
// the gathered weights of rows of 800 inputs within LDS; 64-column slices use all 64.
// (Seven testers: leaving the wavefront that shares the producer's SIMD idle, or 11 or 15 testers,
// measured no faster.)
constexpr int SPLIT_WAVES = 8, SPLIT_TESTERS = SPLIT_WAVES - 1;
constexpr int SPLIT_THREADS = SPLIT_WAVES * kWave;
constexpr int SPLIT_STATIC_LDS = 3 * SPLIT_WAVES * kWave * 4 + 16;
constexpr int SPLIT_SPIN_LIMIT = 1 << 20;                  // default number of polls of the progress counter before a
                                                           // tester gives up (NeuronParams::wait_polls carries the one in force)
// Tester wavefronts that gave up since the process started: one word per device, written (a vector
// atomic) only on that path, read by read_scan_giveups().
__device__ unsigned int g_scan_giveups = 0;
constexpr int SPLIT_PAD = 4;                               // floats between the weight rows of two lanes: the 16-byte
                                                           // reads of eight neighbouring lanes fall on distinct banks
constexpr int SPLIT_ROUND = 4;                             // chunks per round of the producer
constexpr int split_lanes(int cols) { return cols == 64 ? 64 : 32; }

// dynamic LDS of the split kernel: gathered weights [lanes][stride + pad], sorted rows [segs][stride],
// sums after every chunk [chunks + round][2][lanes].  Reads run up to a round past the end of a row
// (into whatever follows, never used); the sums behind the rows keep them inside the allocation.
__host__ __device__ inline size_t split_lds_bytes(int lanes, int segs, int stride) {
    return ((size_t)lanes * (stride + SPLIT_PAD) + (size_t)segs * stride +
            (size_t)(stride / CHUNK + SPLIT_ROUND) * 2 * lanes) * sizeof(float);
}

template <int COLS, bool WANT_K>
__global__ void __launch_bounds__(SPLIT_THREADS)
scan_lds_split_kernel(const float* __restrict__ sorted, const int32_t* __restrict__ perm,
                      const int32_t* __restrict__ n_real, const float* __restrict__ w, float* __restrict__ y_out,
                      float* __restrict__ rcp_out, int32_t* __restrict__ k_out, int S, int I, int stride, int J,
                      int n_slices, int n_groups, NeuronParams np, TimeCopy copy) {
    extern __shared__ __align__(16) float wg[];            // [LANES][stride + SPLIT_PAD], rows, sums
    __shared__ int k_found[SPLIT_WAVES][kWave];
    __shared__ float w_found[SPLIT_WAVES][kWave], y_found[SPLIT_WAVES][kWave];
    __shared__ int progress;                               // chunks whose sums are in LDS
    constexpr int LANES = split_lanes(COLS), SEGS = LANES / COLS;
    constexpr int NONE = 0x7fffffff;
    const int block = xcd_contiguous(blockIdx.x, gridDim.x);
    const int slice = block / n_groups;
    const int group = block - slice * n_groups;
    const int j0 = slice * COLS;
    const int wstride = stride + SPLIT_PAD;
    float* __restrict__ xrows = wg + LANES * wstride;      // [SEGS][stride]
    float* sums = xrows + SEGS * stride;                   // [chunk][wsum|ysum][LANES]

    const int lane = threadIdx.x % kWave;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
    const int la = lane % LANES;                           // lanes past LANES mirror the lower ones
    const int sub = la / COLS, col = la - sub * COLS;
    const int j = j0 + col;
    const float* __restrict__ wrow = wg + la * wstride;
    const float w_bias = np.bias && j < J ? w[(size_t)I * J + j] : 0.0f;

    for (int item = group; item * SEGS < S; item += n_groups) {
        const int seg0 = item * SEGS;
        const int n_segs = S - seg0 < SEGS ? S - seg0 : SEGS;
        const int seg_raw = seg0 + sub;
        // mirror lanes scan along with the lane they mirror (same inputs, same sums, stored to the
        // same place) and only stay out of the output
        const bool scans = seg_raw < S && j < J;
        const bool live = scans && lane < LANES;
        const int seg = seg_raw < S ? seg_raw : S - 1;
        const int row = seg - seg0;                         // idle lanes shadow the item's last segment
        const float* __restrict__ xs = xrows + row * stride;
        const int n = scans ? n_real[seg] : 0;              // (requested before the rows: one round trip less)
        {
            // Weights in scan order: a thread keeps its column and takes four consecutive entries of a
            // row at a time (one 16-byte read of row indices, four weights, one 16-byte LDS write);
            // COLS neighbours read one row of W together.  All row indices of a thread are requested
            // first, then the sorted rows, then all its weights: two memory round trips for the usual
            // item.  (Offsets into W as 24-bit multiply-adds: the launcher checks that rows and row
            // pitch allow it.  Groups past the end repeat the last one.)
            constexpr int KSTEP = SPLIT_THREADS / COLS, GB = 13;
            const int gc = threadIdx.x % COLS, gk = threadIdx.x / COLS;
            const bool col_live = j0 + gc < J;
            const int groups = n_segs * stride / 4;        // stride is a multiple of 16 entries
            const int4* __restrict__ gp = reinterpret_cast<const int4*>(perm + (size_t)seg0 * stride);
            const __amdgpu_buffer_rsrc_t wbuf = __builtin_amdgcn_make_buffer_rsrc(
                const_cast<float*>(w), 0, (int)((size_t)(I + np.bias) * J * sizeof(float)), 0x00020000);
            const unsigned pitch = (unsigned)J * 4u, col_bytes = (unsigned)(j0 + gc) * 4u;
            const int seg_skip = COLS * wstride - stride;  // from entry k of a column to entry k of the next segment
            float* __restrict__ wcol = wg + gc * wstride;
            auto weight = [&](int32_t r) {
                return __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(
                                                     wbuf, __umul24((unsigned)r, pitch) + col_bytes, 0, 0));
            };
            int4 pv[GB];
            auto request_rows = [&](int g0) {
#pragma unroll
                for (int t = 0; t < GB; ++t) pv[t] = gp[min(g0 + t * KSTEP, groups - 1)];
            };
            request_rows(gk);
            __builtin_amdgcn_sched_barrier(0);
            const float4* __restrict__ gx = reinterpret_cast<const float4*>(sorted + (size_t)seg0 * stride);
            for (int e = threadIdx.x; e < groups; e += SPLIT_THREADS) reinterpret_cast<float4*>(xrows)[e] = gx[e];
            for (int g0 = gk;;) {
                float4 wv[GB];
#pragma unroll
                for (int t = 0; t < GB; ++t)
                    wv[t] = col_live ? make_float4(weight(pv[t].x), weight(pv[t].y), weight(pv[t].z), weight(pv[t].w))
                                     : make_float4(0.0f, 0.0f, 0.0f, 0.0f);
#pragma unroll
                for (int t = 0; t < GB; ++t) {
                    const int f = 4 * min(g0 + t * KSTEP, groups - 1);
                    int sl = 0;
#pragma unroll
                    for (int q = 1; q < SEGS; ++q) sl += f >= q * stride;
                    *reinterpret_cast<float4*>(wcol + f + sl * seg_skip) = wv[t];
                }
                g0 += GB * KSTEP;
                if (g0 >= groups) break;
                request_rows(g0);
            }
            if (threadIdx.x == 0) progress = 0;
        }
        __syncthreads();                                    // rows and weights are in place

        const int n_full = n & ~(CHUNK - 1);

        float wsum = -np.theta, ysum = 0.0f, ya = 0.0f;
        bool fired0 = false;
        if (np.bias) {
            wsum += w_bias;
            ysum = np.biasvolt * w_bias;
            ya = wsum < 0.0f ? -ysum : ysum;
            fired0 = ya > fabsf(wsum) * np.biasvolt;
        }
        int k_close = NONE, consumed = 0;
        bool fired_end = false, failed = false;

        if (wave == 0) {
            // ---- producer -----------------------------------------------------------------------
            // chunk c is consumed from buf[c % NBUF]; after it, chunk c + NBUF is read into its place
            constexpr int NBUF = SPLIT_ROUND;
            float bx[NBUF][CHUNK], bw[NBUF][CHUNK];
            auto fetch = [&](float (&x)[CHUNK], float (&wv)[CHUNK], int k) {
                const float4 x0 = *reinterpret_cast<const float4*>(xs + k), x1 = *reinterpret_cast<const float4*>(xs + k + 4);
                const float4 w0 = *reinterpret_cast<const float4*>(wrow + k), w1 = *reinterpret_cast<const float4*>(wrow + k + 4);
                x[0] = x0.x; x[1] = x0.y; x[2] = x0.z; x[3] = x0.w; x[4] = x1.x; x[5] = x1.y; x[6] = x1.z; x[7] = x1.w;
                wv[0] = w0.x; wv[1] = w0.y; wv[2] = w0.z; wv[3] = w0.w; wv[4] = w1.x; wv[5] = w1.y; wv[6] = w1.z; wv[7] = w1.w;
            };
#pragma unroll
            for (int b = 0; b < NBUF; ++b) fetch(bx[b], bw[b], b * CHUNK);
            // chunks of this item: the longest row decides the counter's final value, the shortest how
            // long no lane needs a mask
            int n_full_max = n_full, n_full_min = scans ? n_full : NONE;
#pragma unroll
            for (int d = kWave / 2; d > 0; d >>= 1) {
                n_full_max = max(n_full_max, __shfl_xor(n_full_max, d, kWave));
                n_full_min = min(n_full_min, __shfl_xor(n_full_min, d, kWave));
            }
            n_full_max = __builtin_amdgcn_readfirstlane(n_full_max);
            n_full_min = __builtin_amdgcn_readfirstlane(n_full_min);
            // Order inside a phase: accumulate, store the sums, move the counter to the chunks before
            // this one, then issue the reads for a later chunk.  The counter is a relaxed store and is
            // not waited for: LDS serves a wavefront's requests in order, so the sums it covers, stored
            // a phase earlier, are in place before it.  Nothing moves across a phase boundary (the
            // compiler would otherwise wait for every outstanding request before each accumulation).
            auto publish = [&](int k) {
                asm volatile("" ::: "memory");
                float* out = sums + (k / CHUNK) * 2 * LANES;
                out[la] = wsum;
                out[LANES + la] = ysum;
                asm volatile("" ::: "memory");
                __hip_atomic_store(&progress, k / CHUNK, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
                asm volatile("" ::: "memory");
            };
            int k0 = 0;
            for (; k0 + NBUF * CHUNK <= n_full_min; k0 += NBUF * CHUNK) {
#pragma unroll
                for (int ph = 0; ph < NBUF; ++ph) {
                    const int k = k0 + ph * CHUNK;
                    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                    for (int u = 0; u < CHUNK; ++u) {
                        wsum += bw[ph][u];
                        ysum = __fmaf_rn(bx[ph][u], bw[ph][u], ysum);
                    }
                    publish(k);
                    fetch(bx[ph], bw[ph], k + NBUF * CHUNK);
                }
            }
            for (; k0 < n_full_max; k0 += NBUF * CHUNK) {
#pragma unroll
                for (int ph = 0; ph < NBUF; ++ph) {
                    const int k = k0 + ph * CHUNK;
                    const uint64_t run = __ballot(k < n_full);
                    int unused = 0;
                    __builtin_amdgcn_sched_barrier(0);
                    accumulate_chunk(wsum, ysum, unused, run, bx[ph], bw[ph]);
                    publish(k);
                    fetch(bx[ph], bw[ph], k + NBUF * CHUNK);
                }
            }
            // the last chunk's sums: wait for them, then let the counter reach its final value
            __hip_atomic_store(&progress, (n_full_max + CHUNK - 1) / CHUNK, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_WORKGROUP);
            // the trailing inputs, for a scan that no tester closes
            int kcnt = n_full;
            if (scans) {
                LaneState st;
                st.wsum = wsum; st.ysum = ysum; st.wa = fabsf(wsum);
                st.ya = wsum < 0.0f ? -ysum : ysum;
                st.fired = n_full > 0 ? st.ya > xs[n_full - 1] * st.wa : fired0;
                bool open = true;
                for (int k = n_full; k < n && open; ++k) {
                    open = scan_step(st, xs[k], wrow[k]);
                    if (open) ++kcnt;
                }
                if (!open) k_close = kcnt;
                fired_end = st.fired;
                wsum = st.wsum; ysum = st.ysum;
            }
            k_found[0][lane] = k_close;
            w_found[0][lane] = wsum;
            y_found[0][lane] = ysum;
            consumed = kcnt;                                // all n inputs when nothing closed
        } else {
            // ---- tester t of SPLIT_TESTERS: chunks t, t + SPLIT_TESTERS, ... --------------------------
            uint64_t closed = 0;
            float w_close = 0.0f, y_close = 0.0f;
            float yg = fired0 ? ya : INFINITY;
            float xc[CHUNK], wc[CHUNK], xn[CHUNK], wn[CHUNK];
            auto fetch = [&](float (&x)[CHUNK], float (&wv)[CHUNK], int k) {
                const float4 x0 = *reinterpret_cast<const float4*>(xs + k), x1 = *reinterpret_cast<const float4*>(xs + k + 4);
                const float4 w0 = *reinterpret_cast<const float4*>(wrow + k), w1 = *reinterpret_cast<const float4*>(wrow + k + 4);
                x[0] = x0.x; x[1] = x0.y; x[2] = x0.z; x[3] = x0.w; x[4] = x1.x; x[5] = x1.y; x[6] = x1.z; x[7] = x1.w;
                wv[0] = w0.x; wv[1] = w0.y; wv[2] = w0.z; wv[3] = w0.w; wv[4] = w1.x; wv[5] = w1.y; wv[6] = w1.z; wv[7] = w1.w;
            };
            int c = wave - 1;
            const int last_chunk = stride - CHUNK;
            fetch(xc, wc, c * CHUNK <= last_chunk ? c * CHUNK : 0);
            for (;; c += SPLIT_TESTERS) {
                const int k = c * CHUNK;
                const uint64_t run = __ballot(k < n_full) & ~closed;
                if (run == 0) break;                        // every lane closed here or past its inputs
                const int kn = k + SPLIT_TESTERS * CHUNK;
                fetch(xn, wn, kn <= last_chunk ? kn : 0);
                if (c > 0) {
                    // Bounded wait: if the sums never arrive the tester goes on with what is there and
                    // the result is marked invalid (no early exit: every wavefront reaches the barriers).
                    // The counter and the sums are requested together and waited for once: LDS serves
                    // a wavefront's requests in order, so sums read after a counter that had reached c
                    // are the finished ones; a poll that came too early is repeated as a whole.
                    int spins = 0;
                    const float* in = sums + (c - 1) * 2 * LANES;
                    float x_prev;
                    bool arrived;
                    for (;;) {
                        const int seen = __hip_atomic_load(&progress, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
                        asm volatile("" ::: "memory");
                        wsum = in[la];
                        ysum = in[LANES + la];
                        x_prev = xs[k - 1];
                        asm volatile("" ::: "memory");
                        arrived = __builtin_amdgcn_readfirstlane(seen) >= c;
                        if (arrived || spins >= np.wait_polls) break;
                        __builtin_amdgcn_s_sleep(1);
                        ++spins;
                    }
                    failed |= !arrived;
                    ya = wsum < 0.0f ? -ysum : ysum;        // fired state after input k-1, from the sums
                    yg = ya > x_prev * fabsf(wsum) ? ya : INFINITY;
                }
                const uint64_t before = closed;
                int kc = k;
                scan_chunk_vector<true>(wsum, ysum, ya, yg, kc, closed, run, xc, wc);
                if (((closed & ~before) >> lane) & 1) { k_close = kc; w_close = wsum; y_close = ysum; }
#pragma unroll
                for (int u = 0; u < CHUNK; ++u) { xc[u] = xn[u]; wc[u] = wn[u]; }
            }
            if (failed && lane == 0) atomicAdd(&g_scan_giveups, 1u);
            k_found[wave][lane] = failed ? -1 : k_close;    // -1 poisons the result below
            w_found[wave][lane] = w_close;
            y_found[wave][lane] = y_close;
        }
        __syncthreads();
        if (wave == 0 && live) {
            int best = 0, kb = k_found[0][lane];
            bool bad = false;
#pragma unroll
            for (int v = 1; v < SPLIT_WAVES; ++v) {
                const int kv = k_found[v][lane];
                bad |= kv < 0;
                if (kv < kb) { kb = kv; best = v; }
            }
            // no close anywhere: the producer went through all n inputs, fired_end is the scan's
            const bool fired = kb != NONE || fired_end;
            const float ws = w_found[best][lane], ys = y_found[best][lane];
            float y = np.max_time, r = 0.0f;
            if (fired) {
                r = 1.0f / ws;
                y = ys * r;
                if (y >= np.max_time) { y = np.max_time; r = 0.0f; }
            }
            if (bad) y = r = __builtin_nanf("");            // a tester gave up waiting: make it visible
            const size_t o = (size_t)seg * J + j;
            y_out[o] = y;
            rcp_out[o] = r;
            if (copy.dst) copy.dst[time_copy_pixel(copy, seg) * J + j] = y;
            if (WANT_K) k_out[o] = (fired && r != 0.0f) ? (kb != NONE ? kb : consumed) : -1;
        }
        __syncthreads();                                    // LDS is reused by the next item
    }
}

template <int CH>
__device__ __forceinline__ void read_columns(const float* p, float (&out)[CH]) {
    if constexpr (CH == 1) {
        out[0] = *p;
    } else if constexpr (CH == 2) {
        const float2 v = *reinterpret_cast<const float2*>(p);
        out[0] = v.x; out[1] = v.y;
    } else {
        const float4 v = *reinterpret_cast<const float4*>(p);
        out[0] = v.x; out[1] = v.y; out[2] = v.z; out[3] = v.w;
    }
}
// The same through a pointer that is known to point into LDS.
typedef float lds_float2 __attribute__((ext_vector_type(2)));
template <int CH>
__device__ __forceinline__ void read_columns(__attribute__((address_space(3))) const float* p, float (&out)[CH]) {
    static_assert(CH == 1 || CH == 2, "one or two columns per lane");
    if constexpr (CH == 1) {
        out[0] = *p;
    } else {
        const lds_float2 v = *reinterpret_cast<__attribute__((address_space(3))) const lds_float2*>(p);
        out[0] = v.x; out[1] = v.y;
    }
}

// ---------------------------------------------------------------------------------------------
// Scan with a margin filter: the tests of a step are skipped wherever they provably cannot close.
//
// With D_k = ysum_k - x_k * wsum_k (the state after input k), consuming input k+1 leaves D
// evaluated at x_{k+1} unchanged, and moving from x_k to x_{k+1} changes it by
// -(x_{k+1} - x_k) * wsum_k.  D starts positive (theta * x_0 > 0), rises while wsum < 0 (the
// neuron cannot have fired) and falls while wsum > 0: in exact arithmetic the causal set closes
// at the first step where D reaches zero.  In fp32 the reference's own tests (products rounded
// on their own, sign-corrected compares) can disagree with the sign of D only while |D| is
// within a few ulp of the quantities compared.  So a chunk of eight inputs only accumulates,
//     wsum += w ; ysum = fma(x, w, ysum),
// and is accepted as a whole if t_u = fma(-x_u, wsum_u, ysum_u) is known to lie above
//     thr = 4u * |ysum_end| + 36u * x_last * max|w|        (u = 2^-24)
// after each of its inputs (filter_chunk bounds the eight t from the last one, see there).
// If they all are above thr (and the chunk's first input is not negative) none of the
// reference's tests before the chunk's eight inputs can close the set:
//   * wsum_{k-1} > 0: closing before input k needs ysum_{k-1} <= x_k*wsum_{k-1}*(1+u); the sums
//     after input k differ from those before by the input and two roundings, which puts D_k
//     below u*(3.01*|ysum_k| + x_k*max|w|) / (1 - 2.01u);
//   * wsum_{k-1} < 0: closing needs the neuron fired after input k-1, i.e. D_{k-1} < u*x*|wsum|
//     <= u*(|ysum_{k-1}| + D_{k-1}) -- t of the step before (the last of the previous chunk for
//     the first step; a neuron that fired on its bias alone never takes the fast path);
//   * |ysum| anywhere in the chunk is at most 1.01*(|ysum_end| + 7*x_last*max|w|).
// The running sums are then exactly those of the step-by-step scan, and the fired state is a
// function of them.  A lane whose chunk fails the test keeps the sums it had before the chunk,
// records the chunk and sits out; after the loop every lane evaluates its recorded chunk with
// the reference's tests (the eight-step block above, fed per lane), which finds the close in
// all but contrived cases, and otherwise walks on step by step.  NaN sums never pass a
// reference test and never close; a NaN bound or threshold fails the fast test.
//
// CH (1 or 2) adjacent neurons per lane: one row address and one 4- or 8-byte LDS read serve CH
// scans, and a wavefront covers 64*CH/COLS segments.  Workgroups, slices and items are laid out as
// in scan_lds_kernel, with up to 16 wavefronts per workgroup.
// ---------------------------------------------------------------------------------------------
constexpr float FILTER_REL = 0x1p-22f;                    // 4u
constexpr float FILTER_W = 9.0f * 0x1p-22f;               // 36u, times max|w| of the slice
// The fast loop does not evaluate the eight t of a chunk: it bounds them from the last one.  With the
// sums as computed, D_u = ysum_u - x_u*wsum_u obeys  D_{u-1} = D_u + (x_u - x_{u-1})*wsum_{u-1} - e_u,
// |e_u| <= u*(|ysum_u| + x_u*|wsum_u|) (the roundings of the two sums), hence for every u of the chunk
//     D_u >= D_7 + (x_7 - x_0) * min(0, wsum_0 .. wsum_7) - 7 * max|e|:
// D only falls while the weight sum is positive, and where the sum is negative it can have been lower
// earlier by at most that much.  The lane keeps the smallest weight sum of the chunk (one three-way
// minimum per two inputs, started at zero), evaluates t_7 and accepts the chunk if
//     fma(x_7 - x_0, min, t_7)  >  thr + 12u * 1.01 * (|ysum_7| + x_7*|wsum_7| + 14*x_7*max|w|)
// (the second term covers the seven e_u, the roundings of t_u, t_7, x_7 - x_0 and of the bound itself;
// sums inside the chunk differ from the final ones by at most seven inputs).  Every t_u then exceeds
// thr, which is the condition above.  With a weight sum that stays positive the bound is t_7 itself, so
// a chunk fails exactly where it failed before, give or take the wider margin (a few 10^-6 of the sums).
// Two additions, one half of a minimum per input instead of three and a half instructions.
constexpr float FILTER_END_Y = 0x1p-19f;                  // 32u >= 4u + 12.2u, times |ysum_7|
constexpr float FILTER_END_XW = 0x1p-20f;                 // 16u >= 12.2u, times x_7 * |wsum_7|
constexpr float FILTER_END_W = 0x1p-16f;                  // 256u >= 36u + 170u, times x_7 * max|w| of the slice

// Eight inputs for one scan of every lane.  Lanes in the mask `open` that pass the test keep the new
// sums; open lanes that fail keep the old ones, take the chunk's first index as kflag and leave
// `open`.  The arithmetic does not depend on EXEC or branches (lanes that are not open compute along
// and discard), so the compiler is free to interleave it with the LDS traffic of the next chunk; the
// decision works on lane masks in scalar registers: one compare, three mask operations, three selects.
// dx = x[7] - x[0], x7s = FILTER_END_XW * x[7], thrx = FILTER_END_W * max|w| * x[7].
__device__ __forceinline__ void filter_chunk(float& wsum, float& ysum, int& kflag, uint64_t& open, int k, float thrx,
                                             float dx, float x7s, const float (&x)[CHUNK], const float (&w)[CHUNK]) {
    float wb = wsum, yb = ysum, m = 0.0f;
#pragma unroll
    for (int u = 0; u < CHUNK; u += 2) {
        wb += w[u];
        yb = __fmaf_rn(x[u], w[u], yb);
        const float w0 = wb;
        wb += w[u + 1];
        yb = __fmaf_rn(x[u + 1], w[u + 1], yb);
        m = fminf(fminf(m, w0), wb);
    }
    const float t7 = __fmaf_rn(-x[CHUNK - 1], wb, yb);
    const float bound = __fmaf_rn(dx, m, t7);
    const float thr = __fmaf_rn(FILTER_END_Y, fabsf(yb), __fmaf_rn(x7s, fabsf(wb), thrx));
    uint64_t stop;
    // (two statements: the first has scalar results only, so the masks stay uniform values for the compiler
    // also where no branch depends on them)
    asm("v_cmp_gt_f32_e32 vcc, %[m], %[thr]\n"                       // pass: false for NaN on either side
        "s_andn2_b64 %[stop], %[open], vcc\n"
        "s_and_b64 %[open], %[open], vcc\n"
        : [open] "+s"(open), [stop] "=&s"(stop)
        : [m] "v"(bound), [thr] "v"(thr)
        : "vcc", "scc");
    asm("v_cndmask_b32_e64 %[ws], %[ws], %[wb], %[open]\n"
        "v_cndmask_b32_e64 %[ys], %[ys], %[yb], %[open]\n"
        "v_cndmask_b32_e64 %[kf], %[kf], %[vk], %[stop]\n"
        : [ws] "+v"(wsum), [ys] "+v"(ysum), [kf] "+v"(kflag)
        : [open] "s"(open), [stop] "s"(stop), [wb] "v"(wb), [yb] "v"(yb), [vk] "v"(k));
}

// Largest of the threads' `m` over the workgroup, the same value in every thread.  `red` is room for
// one float per wavefront; the call contains the workgroup barrier that also publishes whatever the
// threads wrote to LDS before it.
__device__ __forceinline__ float block_max(float m, float* __restrict__ red) {
#pragma unroll
    for (int d = kWave / 2; d > 0; d >>= 1) m = fmaxf(m, __shfl_xor(m, d, kWave));
    if (threadIdx.x % kWave == 0) red[threadIdx.x / kWave] = m;
    __syncthreads();
    const int waves = blockDim.x / kWave;
    float r = red[0];
    for (int v = 1; v < waves; ++v) r = fmaxf(r, red[v]);
    return r;
}

constexpr int FILTER_RED_BYTES = 64;                       // one float per wavefront behind the slice

// Value of `v` in lane 4*(lane/4) + q: a quad broadcast, which the hardware applies as an operand
// modifier (DPP) of the move or of the VOP2 instruction that consumes it.
template <int Q>
__device__ __forceinline__ int quad_broadcast(int v) {
    return __builtin_amdgcn_mov_dpp(v, Q * 0x55, 0xf, 0xf, true);
}

// a[q] = base + (value of `row` in lane q of the quad << SHIFT), q = 0..3: the LDS addresses of four
// weight rows from the row indices the quad's lanes hold.  One shift, then four adds that take the
// broadcast as an operand modifier (the two idle cycles between them are what a DPP read of a
// register written by the instruction before it needs).
template <int SHIFT>
__device__ __forceinline__ void quad_row_addresses(int row, unsigned base, unsigned (&a)[4]) {
    int t;
    asm("v_lshlrev_b32_e32 %[t], %[sh], %[row]\n"
        "s_nop 1\n"
        "v_add_u32_dpp %[a0], %[t], %[base] quad_perm:[0,0,0,0] row_mask:0xf bank_mask:0xf bound_ctrl:1\n"
        "v_add_u32_dpp %[a1], %[t], %[base] quad_perm:[1,1,1,1] row_mask:0xf bank_mask:0xf bound_ctrl:1\n"
        "v_add_u32_dpp %[a2], %[t], %[base] quad_perm:[2,2,2,2] row_mask:0xf bank_mask:0xf bound_ctrl:1\n"
        "v_add_u32_dpp %[a3], %[t], %[base] quad_perm:[3,3,3,3] row_mask:0xf bank_mask:0xf bound_ctrl:1\n"
        : [t] "=&v"(t), [a0] "=&v"(a[0]), [a1] "=&v"(a[1]), [a2] "=&v"(a[2]), [a3] "=&v"(a[3])
        : [row] "v"(row), [base] "v"(base), [sh] "n"(SHIFT));
}

typedef __attribute__((address_space(3))) const float lds_cfloat;

// f(integral_constant<int, 0>), f(<1>), ... f(<N-1>) until one returns false; true if none did.  The
// phase number reaches f as a type, so ring slots and buffers stay compile-time register choices.
template <class F, int... PH>
__device__ __forceinline__ bool for_each_phase_impl(F&& f, std::integer_sequence<int, PH...>) {
    return (f(std::integral_constant<int, PH>{}) && ...);
}
template <int N, class F>
__device__ __forceinline__ bool for_each_phase(F&& f) {
    return for_each_phase_impl(f, std::make_integer_sequence<int, N>{});
}

// Segments a wavefront of the filter kernel works on, and whether their input times go through
// LDS: they do unless every quad has a segment of its own (then the quad broadcast is all there is
// to share, and the buffers of 16 segments per wavefront would not fit beside the slice).
constexpr int filter_segments(int cols, int ch) { return kWave / (cols / ch); }
constexpr bool filter_stages_times(int cols, int ch) { return filter_segments(cols, ch) <= 8; }
// dynamic LDS of a workgroup of `waves` wavefronts behind its slice
constexpr size_t filter_extra_lds(int cols, int ch, int waves) {
    return FILTER_RED_BYTES + (filter_stages_times(cols, ch) ? (size_t)waves * filter_segments(cols, ch) * FILTER_XBUF_SEG_BYTES : 0);
}

template <int COLS, int CH, bool WANT_K>
__global__ void __launch_bounds__(LDS_SCAN_THREADS)
scan_filter_kernel(const float* __restrict__ sorted, const int32_t* __restrict__ perm,
                   const int32_t* __restrict__ n_real, const float* __restrict__ w, float* __restrict__ y_out,
                   float* __restrict__ rcp_out, int32_t* __restrict__ k_out, int S, int I, int stride, int J,
                   int n_slices, int n_groups, NeuronParams np, TimeCopy copy) {
    extern __shared__ __align__(16) float wl[];                          // [I + bias][COLS], then `red`
    constexpr int LANES = COLS / CH;                       // lanes per segment
    constexpr int SEGS = kWave / LANES;                    // segments per wavefront
    static_assert(LANES % 4 == 0, "the four lanes of a quad belong to one segment");
    // Input times reach the lanes through LDS where several quads share a segment (see the fast loop)
    constexpr bool XLDS = filter_stages_times(COLS, CH);
    const int WAVES = blockDim.x / kWave;
    const int block = xcd_contiguous(blockIdx.x, gridDim.x);
    const int slice = block / n_groups;
    const int group = block - slice * n_groups;
    const int j0 = slice * COLS;
    const int rows = I + np.bias;
    // the slice, and the largest |w| in it (the threads' shares of the copy, then the workgroup's)
    const float w_max = block_max(fill_weight_slice<COLS>(wl, w, rows, J, j0), wl + rows * COLS);
    const float thr_w = FILTER_W * w_max;                   // margin of the accumulate-only rounds below
    const float end_w = FILTER_END_W * w_max;               // margin of the fast loop

    const int lane = threadIdx.x % kWave;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
    const int sub = lane / LANES, cg = lane - sub * LANES;
    const int j = j0 + CH * cg;                            // first of the lane's columns
    const float* __restrict__ wcol = wl + CH * cg;
    const int last_chunk = stride - CHUNK;

    const int quad_lane = lane & 3;
    const unsigned wbase = (unsigned)(uintptr_t)(lds_cfloat*)wcol;          // LDS byte address of the lane's columns
    // [wave][buffer][segment of the wavefront][CHUNK] input times, behind the slice and `red`
    float* __restrict__ xbuf = wl + rows * COLS + FILTER_RED_BYTES / (int)sizeof(float) +
                               (size_t)wave * 2 * SEGS * CHUNK + sub * CHUNK;
    const bool x_writer = cg < 4;                          // the first quad of every segment
    constexpr int NONE = 0x7fffffff;
    constexpr int ROW_SHIFT = COLS == 64 ? 8 : COLS == 32 ? 7 : COLS == 16 ? 6 : 5;      // a weight row is COLS * 4 bytes
    static_assert(COLS == 64 || COLS == 32 || COLS == 16 || COLS == 8, "slice width");

    for (int item = group * WAVES + wave; item * SEGS < S; item += n_groups * WAVES) {
        const int seg_raw = item * SEGS + sub;
        const int seg = seg_raw < S ? seg_raw : S - 1;      // idle lanes shadow a valid segment
        const float* __restrict__ xs = sorted + (size_t)seg * stride;
        const int32_t* __restrict__ pr = perm + (size_t)seg * stride;
        const int seg0 = __builtin_amdgcn_readfirstlane(item * SEGS);
        const int n_segs = S - seg0 < SEGS ? S - seg0 : SEGS;
        const RowSource rows_of_item = make_row_source(sorted + (size_t)seg0 * stride, perm + (size_t)seg0 * stride,
                                                       n_segs * stride * (int)sizeof(float));
        const int lane_bytes = ((seg - seg0) * stride + quad_lane) * (int)sizeof(float);
        const int n_seg = n_real[seg];
        const float first_x = xs[0];
        // The ring of (x, row) entries the fast loop below consumes (see there).  Its first round is requested
        // here, next to the two loads above and before anything waits for them: practically every item
        // starts its first pass at input 0, and the round trips would otherwise follow one another.
        constexpr int RING = 8;                             // chunks of entries held or on their way
        float rxl[RING], rxh[RING];
        int rpl[RING], rph[RING];
        auto request = [&](int slot, int k) {
            const int kb = (k <= last_chunk ? k : 0) * (int)sizeof(float);
            rxl[slot] = __uint_as_float(__builtin_amdgcn_raw_buffer_load_b32(rows_of_item.xs, lane_bytes, kb, 0));
            rxh[slot] = __uint_as_float(__builtin_amdgcn_raw_buffer_load_b32(rows_of_item.xs, lane_bytes + 16, kb, 0));
            rpl[slot] = (int)__builtin_amdgcn_raw_buffer_load_b32(rows_of_item.pr, lane_bytes, kb, 0);
            rph[slot] = (int)__builtin_amdgcn_raw_buffer_load_b32(rows_of_item.pr, lane_bytes + 16, kb, 0);
        };
#pragma unroll
        for (int b = 0; b < RING - 1; ++b) request(b, b * CHUNK);
        bool ring_at_zero = true;                           // the ring holds the entries from input 0 on
        const int n_full = n_seg & ~(CHUNK - 1);

        // Per scan: the running sums, the number of inputs they hold (kcur), and where the scan stands:
        //   armed    waits to run the fast loop from kcur (no reference test can close before kcur)
        //   kflag    first index of a chunk that failed the fast test and has to be stepped through (or -1)
        //   fin      closed; sums, fired state and count are final
        float wsum[CH], ysum[CH];
        int kcur[CH], kflag[CH];
        bool live[CH], armed[CH], fin[CH], fired_cur[CH];   // fired_cur: the fired state that goes with the sums
        float wb[CH];
        if (np.bias) read_columns<CH>(wcol + I * COLS, wb);
#pragma unroll
        for (int c = 0; c < CH; ++c) {
            live[c] = seg_raw < S && j + c < J;
            wsum[c] = -np.theta; ysum[c] = 0.0f;
            fired_cur[c] = false;
            if (np.bias) {
                wsum[c] += wb[c];
                ysum[c] = np.biasvolt * wb[c];
                const float ya0 = wsum[c] < 0.0f ? -ysum[c] : ysum[c];
                fired_cur[c] = ya0 > fabsf(wsum[c]) * np.biasvolt;
            }
            kcur[c] = 0;
            fin[c] = false;
            // The fast loop takes scans whose fired state is what their sums imply between tests that
            // pass with a margin: fired exactly when the weight sum is positive, and whose remaining
            // inputs are not negative (its bounds assume x >= 0; rows are ascending).  Any other start (a
            // neuron that fired on its bias alone, a row that begins below zero) is stepped through
            // from the first input on.
            const bool plain = fired_cur[c] == (wsum[c] > 0.0f) && !fired_cur[c] && first_x >= 0.0f;
            armed[c] = live[c] && n_full > 0 && plain;
            kflag[c] = (live[c] && n_full > 0 && !plain) ? 0 : -1;
        }

        // Passes: the fast loop for the armed scans that are furthest behind, then the recorded
        // chunks step by step.  A scan that does not close in its recorded chunk is armed again.
        // Practically every item takes one pass and a second look without work.
        bool first_pass = true;
        for (;;) {
            int kmin = NONE;
#pragma unroll
            for (int c = 0; c < CH; ++c) kmin = armed[c] ? min(kmin, kcur[c]) : kmin;
            if (first_pass) {                               // every armed scan starts at input 0
                kmin = __builtin_amdgcn_ballot_w64(kmin != NONE) != 0 ? 0 : NONE;
            } else {
#pragma unroll
                for (int d = kWave / 2; d > 0; d >>= 1) kmin = min(kmin, __shfl_xor(kmin, d, kWave));
                kmin = __builtin_amdgcn_readfirstlane(kmin);
            }
            first_pass = false;
            if (kmin != NONE) {
                uint64_t open[CH];                          // lanes whose scan runs in this loop
                bool ran[CH];
#pragma unroll
                for (int c = 0; c < CH; ++c) {
                    ran[c] = armed[c] && kcur[c] == kmin;
                    open[c] = __builtin_amdgcn_ballot_w64(ran[c]);
                    armed[c] = armed[c] && !ran[c];
                    kcur[c] = ran[c] ? n_full : kcur[c];    // unless the scan records a chunk below
                }
                // The (x, row) stream of a segment is the same for all its lanes.  If every lane fetched
                // the eight entries of a chunk itself, a wavefront would move four kilobytes per chunk
                // through the vector memory path, which then bounds the kernel.  Instead the four lanes
                // of a quad fetch entries q and q + 4 of both arrays (q = lane % 4: four dwords per lane
                // and chunk, through buffer loads that need no address arithmetic), and a value reaches
                // the other lanes of the quad as a quad broadcast: free for the row offsets, which enter
                // the LDS address through an add that takes the broadcast as an operand modifier, one
                // move per input time (shared by the lane's CH scans).
                // Per phase, with c the chunk being consumed: request the entries of chunk c+RING-1, read
                // the weights of chunk c+1 from LDS, run chunk c.
                float wv[2][CH][CHUNK];                     // [buffer][scan][step]
                auto weights = [&](int slot, float (&wo)[CH][CHUNK]) {
                    unsigned al[4], ah[4];
                    quad_row_addresses<ROW_SHIFT>(rpl[slot], wbase, al);
                    quad_row_addresses<ROW_SHIFT>(rph[slot], wbase, ah);
#pragma unroll
                    for (int u = 0; u < CHUNK; ++u) {
                        float wr[CH];
                        read_columns<CH>(reinterpret_cast<lds_cfloat*>((uintptr_t)(u < 4 ? al[u] : ah[u - 4])), wr);
#pragma unroll
                        for (int c = 0; c < CH; ++c) wo[c][u] = wr[c];
                    }
                };
                // Input times: with DPP alone every lane needs a move per time and chunk.  Where a
                // segment spans several quads, its first quad instead leaves the eight times of the
                // next chunk in a small LDS buffer of the wavefront (two chunks deep) and every lane
                // reads them back as two 16-byte broadcasts, a phase ahead like the weights.  LDS
                // serves the requests of a wavefront in order, so the reads find what was written.
                float xq[2][CHUNK];
                auto stage_times = [&](int slot, int buf) {
                    if constexpr (XLDS) {
                        float* __restrict__ xb = xbuf + buf * SEGS * CHUNK;
                        if (x_writer) {
                            xb[quad_lane] = rxl[slot];
                            xb[quad_lane + 4] = rxh[slot];
                        }
                        __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
                        __builtin_amdgcn_wave_barrier();
                        const float4 lo = *reinterpret_cast<const float4*>(xb), hi = *reinterpret_cast<const float4*>(xb + 4);
                        xq[buf][0] = lo.x; xq[buf][1] = lo.y; xq[buf][2] = lo.z; xq[buf][3] = lo.w;
                        xq[buf][4] = hi.x; xq[buf][5] = hi.y; xq[buf][6] = hi.z; xq[buf][7] = hi.w;
                    }
                };
                if (!(ring_at_zero && kmin == 0)) {
#pragma unroll
                    for (int b = 0; b < RING - 1; ++b) request(b, kmin + b * CHUNK);
                }
                ring_at_zero = false;
                weights(0, wv[0]);
                // (every lane "uses" the first chunk's times here: otherwise the compiler moves their loads
                // under the writers' branch of stage_times and waits for all 28 requests there)
                if constexpr (XLDS) asm volatile("" : "+v"(rxl[0]), "+v"(rxh[0]));
                stage_times(0, 0);

                // One phase; its number is a compile-time value.  (The phases of a round are chained by a fold
                // expression, not by a loop with a break: behind such a loop the compiler waits in every
                // phase for all but the last four row loads, which makes the ring one chunk deep in effect.)
                auto phase = [&](auto ph_c, int k) {
                    constexpr int ph = decltype(ph_c)::value;
                    request((ph + RING - 1) % RING, k + (RING - 1) * CHUNK);
                    weights((ph + 1) % RING, wv[(ph + 1) % 2]);
                    stage_times((ph + 1) % RING, (ph + 1) % 2);
                    // The requests above stay ahead of the arithmetic below: what this phase consumes
                    // was requested a phase or more ago, and what it requests has the whole phase to
                    // arrive.
                    __builtin_amdgcn_sched_barrier(0);
                    float x[CHUNK];
                    if constexpr (XLDS) {
#pragma unroll
                        for (int u = 0; u < CHUNK; ++u) x[u] = xq[ph % 2][u];
                    } else {
                        const int xl = __float_as_int(rxl[ph % RING]), xh = __float_as_int(rxh[ph % RING]);
                        x[0] = __int_as_float(quad_broadcast<0>(xl)); x[1] = __int_as_float(quad_broadcast<1>(xl));
                        x[2] = __int_as_float(quad_broadcast<2>(xl)); x[3] = __int_as_float(quad_broadcast<3>(xl));
                        x[4] = __int_as_float(quad_broadcast<0>(xh)); x[5] = __int_as_float(quad_broadcast<1>(xh));
                        x[6] = __int_as_float(quad_broadcast<2>(xh)); x[7] = __int_as_float(quad_broadcast<3>(xh));
                    }
                    const float thrx = x[CHUNK - 1] * end_w, x7s = x[CHUNK - 1] * FILTER_END_XW;
                    const float dx = x[CHUNK - 1] - x[0];
#pragma unroll
                    for (int c = 0; c < CH; ++c)
                        filter_chunk(wsum[c], ysum[c], kflag[c], open[c], k, thrx, dx, x7s, x, wv[ph % 2][c]);
                };
                for (int k0 = kmin;; k0 += RING * CHUNK) {
                    rotate_wave_priority(k0 / (RING * CHUNK) + (wave >> 2));
                    const bool stop = !for_each_phase<RING>([&](auto ph_c) {
                        const int k = k0 + decltype(ph_c)::value * CHUNK;
                        const uint64_t inside = __builtin_amdgcn_ballot_w64(k < n_full);
                        uint64_t any = 0;
#pragma unroll
                        for (int c = 0; c < CH; ++c) {
                            open[c] &= inside;
                            any |= open[c];
                        }
                        if (any == 0) return false;
                        phase(ph_c, k);
                        return true;
                    });
                    if (stop) break;
                }
#pragma unroll
                for (int c = 0; c < CH; ++c) fired_cur[c] = ran[c] ? wsum[c] > 0.0f : fired_cur[c];
            }

            // Recorded chunks, stepped through with the reference's tests: every lane fetches its own
            // eight inputs (positions are multiples of eight inside the full chunks of the row).  A scan
            // that closes is finished.  One that does not goes back to the fast loop if its fired state is
            // the plain one; otherwise (fired on a negative weight sum, say) it keeps stepping here, chunk
            // by chunk.
            bool need[CH], any_need = false, any_armed = false;
            Chunk pc[CH];
#pragma unroll
            for (int c = 0; c < CH; ++c) {
                need[c] = kflag[c] >= 0;
                kcur[c] = need[c] ? kflag[c] : kcur[c];
                kflag[c] = -1;
                any_need |= need[c];
                any_armed |= armed[c];
            }
            if (__builtin_amdgcn_ballot_w64(any_need) != 0) {
                int round = 0;
                do {
                    // (fetched on demand: a second round is rare, requesting its entries ahead of time
                    // would cost every item eight more loads per scan)
#pragma unroll
                    for (int c = 0; c < CH; ++c) load_chunk_flat(pc[c], xs, pr, need[c] ? kcur[c] : 0);
                    any_need = false;
#pragma unroll
                    for (int c = 0; c < CH; ++c) {
                        float pw[CHUNK], px[CHUNK];
#pragma unroll
                        for (int u = 0; u < CHUNK; ++u) {
                            pw[u] = wcol[pc[c].p[u] * COLS + c];
                            px[u] = pc[c].x[u];
                        }
                        // Later rounds are for the rare scan that missed its close by a rounding: weight
                        // sum positive, not fired (D < 0).  It cannot fire, let alone close, before the
                        // weight sum has been negative long enough for D to come back up to zero, and it
                        // walks on here, a chunk per round, usually in a wavefront that is alone by then.
                        // While every scan of the round is in that state, a chunk is only accumulated and
                        // bounded: with all t = ysum - x*wsum below -thr (the fast loop's margin) and all
                        // weight sums positive, the reference's `fired` test is false after each of the
                        // eight inputs, and that is all it evaluates for a scan that has not fired.
                        bool walked = false;
                        if (round > 0) {
                            const bool stuck = need[c] && !fired_cur[c] && wsum[c] > 0.0f && px[0] >= 0.0f;
                            if (__builtin_amdgcn_ballot_w64(need[c] && !stuck) == 0) {
                                float wb = wsum[c], yb = ysum[c], tmax = -INFINITY, wmin = INFINITY;
#pragma unroll
                                for (int u = 0; u < CHUNK; ++u) {
                                    wb += pw[u];
                                    yb = __fmaf_rn(px[u], pw[u], yb);
                                    tmax = fmaxf(tmax, __fmaf_rn(-px[u], wb, yb));
                                    wmin = fminf(wmin, wb);
                                }
                                const float thr = __fmaf_rn(FILTER_REL, fabsf(yb), px[CHUNK - 1] * thr_w);
                                walked = stuck && tmax < -thr && wmin > 0.0f;
                                wsum[c] = walked ? wb : wsum[c];
                                ysum[c] = walked ? yb : ysum[c];
                            }
                        }
                        float ya = wsum[c] < 0.0f ? -ysum[c] : ysum[c];
                        float yg = fired_cur[c] ? ya : INFINITY;
                        uint64_t exited = 0;
                        int kc = kcur[c] + (walked ? CHUNK : 0);
                        const uint64_t run = __builtin_amdgcn_ballot_w64(need[c] && !walked);
                        if (run != 0) scan_chunk_vector<true>(wsum[c], ysum[c], ya, yg, kc, exited, run, px, pw);
                        const bool closed_here = (exited >> lane) & 1;
                        kcur[c] = kc;                       // inputs consumed
                        fin[c] = fin[c] || closed_here;
                        fired_cur[c] = closed_here || yg < INFINITY;
                        const bool more = need[c] && !closed_here && kc + CHUNK <= n_full;
                        const bool plain = fired_cur[c] == (wsum[c] > 0.0f) && px[CHUNK - 1] >= 0.0f;
                        armed[c] = armed[c] || (more && plain);
                        any_armed |= more && plain;
                        need[c] = more && !plain;
                        any_need |= need[c];
                    }
                    ++round;
                } while (__builtin_amdgcn_ballot_w64(any_need) != 0);
            }
            if (__builtin_amdgcn_ballot_w64(any_armed) == 0) break;
        }

        // Whatever is left of a row -- fewer than eight inputs behind the full chunks -- step by step,
        // then the output.  The leftover entries and their weights are fetched in one go for the
        // lane's CH scans (a load per step would put a memory round trip into every one of them); rows
        // are padded beyond their length, so the eight entries from n_full on can always be read.
        LaneState st[CH];
        int kc[CH];
        bool still[CH], any_left = false;
#pragma unroll
        for (int c = 0; c < CH; ++c) {
            st[c].wsum = wsum[c]; st[c].ysum = ysum[c]; st[c].wa = fabsf(wsum[c]);
            st[c].ya = wsum[c] < 0.0f ? -ysum[c] : ysum[c];
            st[c].fired = fired_cur[c];
            kc[c] = kcur[c];
            still[c] = live[c] && !fin[c];
            any_left |= still[c] && kc[c] < n_seg;
        }
        if (__builtin_amdgcn_ballot_w64(any_left) != 0) {
            Chunk tc;
            load_chunk_flat(tc, xs, pr, n_full < n_seg ? n_full : 0);
            float tw[CH][CHUNK];
#pragma unroll
            for (int c = 0; c < CH; ++c)
#pragma unroll
                for (int u = 0; u < CHUNK; ++u) tw[c][u] = wcol[tc.p[u] * COLS + c];
#pragma unroll
            for (int u = 0; u < CHUNK - 1; ++u) {
                bool any_step = false;
#pragma unroll
                for (int c = 0; c < CH; ++c) {
                    const bool step = still[c] && kc[c] == n_full + u && n_full + u < n_seg;
                    if (step) {
                        still[c] = scan_step(st[c], tc.x[u], tw[c][u]);
                        if (still[c]) ++kc[c];
                    }
                    any_step |= step;
                }
                if (__builtin_amdgcn_ballot_w64(any_step) == 0) break;
            }
        }
#pragma unroll
        for (int c = 0; c < CH; ++c) {
            if (!live[c]) continue;
            // (a scan that stands before the full chunks' end here does not occur; it would be walked like this)
            for (int k = kc[c]; k < n_seg && still[c]; ++k) {
                still[c] = scan_step(st[c], xs[k], wcol[pr[k] * COLS + c]);
                if (still[c]) ++kc[c];
            }
            float y = np.max_time, r = 0.0f;
            if (st[c].fired) {
                r = 1.0f / st[c].wsum;
                y = st[c].ysum * r;
                if (y >= np.max_time) { y = np.max_time; r = 0.0f; }
            }
            const size_t o = (size_t)seg * J + j + c;
            y_out[o] = y;
            rcp_out[o] = r;
            if (copy.dst) copy.dst[time_copy_pixel(copy, seg) * J + j + c] = y;
            if (WANT_K) k_out[o] = (st[c].fired && r != 0.0f) ? kc[c] : -1;
        }
    }
}

__global__ void __launch_bounds__(256)
unpad_rows_kernel(const float* __restrict__ sorted, const int32_t* __restrict__ perm,
                  float* __restrict__ sorted_out, int32_t* __restrict__ perm_out, int64_t n, int I, int stride) {
    const int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (t >= n) return;
    const int64_t row = t / I;
    const int col = (int)(t - row * I);
    const size_t src = (size_t)row * stride + col;
    if (sorted_out) sorted_out[t] = sorted[src];
    if (perm_out) perm_out[t] = perm[src];
}

}  // namespace

namespace {
// Neurons per lane of the instantiation for large launches: two (four need 151 registers: too few
// wavefronts per SIMD, measured slower), except with 8-column slices, whose 32-byte weight rows make
// the 8-byte reads of two-neuron lanes collide in the LDS banks (sixteen rows per read on four bank
// groups): one neuron per lane reads eight rows at 4 bytes a lane.
constexpr int filter_ch(int cols) { return cols == 8 ? 1 : 2; }

template <int COLS>
int raise_scan_lds_limits() {
    const void* whole[] = {
        reinterpret_cast<const void*>(scan_lds_kernel<COLS, true>),
        reinterpret_cast<const void*>(scan_lds_kernel<COLS, false>),
        reinterpret_cast<const void*>(scan_filter_kernel<COLS, 1, true>),
        reinterpret_cast<const void*>(scan_filter_kernel<COLS, 1, false>),
        reinterpret_cast<const void*>(scan_filter_kernel<COLS, filter_ch(COLS), true>),
        reinterpret_cast<const void*>(scan_filter_kernel<COLS, filter_ch(COLS), false>)};
    for (const void* k : whole)
        SNNTC_HIP_CHECK(hipFuncSetAttribute(k, hipFuncAttributeMaxDynamicSharedMemorySize, LDS_SCAN_BYTES));
    const void* split[] = {reinterpret_cast<const void*>(scan_lds_split_kernel<COLS, true>),
                           reinterpret_cast<const void*>(scan_lds_split_kernel<COLS, false>)};
    for (const void* k : split)
        SNNTC_HIP_CHECK(hipFuncSetAttribute(k, hipFuncAttributeMaxDynamicSharedMemorySize,
                                            LDS_SCAN_BYTES - SPLIT_STATIC_LDS));
    return SNNTC_OK;
}
}  // namespace

// One-time set-up of the scan on device `dev` (which must be the current device): the CU count and
// the dynamic-LDS limit of EVERY instantiation, so that no later launch, whatever its shape, has
// to call hipFuncSetAttribute (which is not allowed while a stream is being captured).
int scan_prepare_device(int dev, int* cu_count_out) {
    static std::atomic<int> cu_count[kMaxDevices];
    if (dev < 0 || dev >= kMaxDevices) return fail(SNNTC_ERR_UNSUPPORTED, "scan: device index %d not supported", dev);
    int cus = cu_count[dev].load(std::memory_order_acquire);
    if (cus == 0) {
        hipDeviceProp_t prop;
        SNNTC_HIP_CHECK(hipGetDeviceProperties(&prop, dev));
        int rc = raise_scan_lds_limits<64>();
        if (!rc) rc = raise_scan_lds_limits<32>();
        if (!rc) rc = raise_scan_lds_limits<16>();
        if (!rc) rc = raise_scan_lds_limits<8>();
        if (rc) return rc;
        cus = prop.multiProcessorCount > 0 ? prop.multiProcessorCount : 256;
        cu_count[dev].store(cus, std::memory_order_release);
    }
    if (cu_count_out) *cu_count_out = cus;
    return SNNTC_OK;
}

namespace {
std::atomic<int> g_wait_polls{SPLIT_SPIN_LIMIT};
}

void set_scan_wait_polls(int polls) { g_wait_polls.store(polls < 0 ? SPLIT_SPIN_LIMIT : polls, std::memory_order_relaxed); }

int read_scan_giveups(int64_t* count, hipStream_t stream) {
    unsigned int v = 0;
    SNNTC_HIP_CHECK(hipMemcpyFromSymbolAsync(&v, HIP_SYMBOL(g_scan_giveups), sizeof(v), 0, hipMemcpyDeviceToHost, stream));
    SNNTC_HIP_CHECK(hipStreamSynchronize(stream));
    *count = (int64_t)v;
    return SNNTC_OK;
}

template <int COLS>
int launch_scan_lds(const float* sorted, const int32_t* perm, const int32_t* n_real, const float* w, float* y,
                    float* rcp, int32_t* causal_k, int64_t S, int64_t I, int64_t stride, int64_t J,
                    const NeuronParams& np_in, const TimeCopy& copy, size_t lds_bytes, hipStream_t stream) {
    NeuronParams np = np_in;
    np.wait_polls = g_wait_polls.load(std::memory_order_relaxed);
    int dev = 0, cus = 0;
    SNNTC_HIP_CHECK(hipGetDevice(&dev));
    const int prep = scan_prepare_device(dev, &cus);
    if (prep) return prep;
    constexpr int SEGS = kWave / COLS;
    const int n_slices = (int)((J + COLS - 1) / COLS);
    const int64_t items = (S + SEGS - 1) / SEGS;
    // workgroups the chip holds at once (two per CU when two weight slices fit in its LDS)
    const int wgs_per_cu = (lds_bytes + filter_extra_lds(COLS, 1, 16)) * 2 <= (size_t)LDS_SCAN_BYTES ? 2 : 1;
    const int64_t capacity = (int64_t)cus * wgs_per_cu;
    // A launch whose work items all find a wavefront of their own in workgroups of four (one
    // wavefront per SIMD of a CU, and four times the threads of a single wavefront for copying the
    // weight slice) runs the low-latency instantiation: the same work packed into a few full
    // workgroups would leave most of the chip idle.  Larger launches get the workgroup size, 4 to
    // 16 wavefronts, that spreads them over all CUs in one go.
    const bool low_latency = (items + 3) / 4 * n_slices <= capacity;
    int WAVES = LOW_LATENCY_THREADS / kWave;
    if (!low_latency) {
        const int64_t per_wg = (items * n_slices + capacity - 1) / capacity;
        WAVES = (int)(per_wg >= 16 ? 16 : (per_wg + 3) / 4 * 4);
    }
    // With at least four wavefronts of multi-neuron lanes for every SIMD, CH neurons per lane (CH times
    // the segments per wavefront) is the cheaper instruction stream; in between, one neuron per
    // lane in 16-wave workgroups balances better -- as long as those workgroups fit the chip in one
    // go: once one-neuron lanes would need a second round of workgroups, the multi-neuron form, which
    // still fits, is the faster one (800 x 800 at B = 384: 55 against 79 us).
    constexpr int CH = filter_ch(COLS);
    const int64_t multi_items = (S + CH * SEGS - 1) / (CH * SEGS);
    const bool multi = !low_latency && (multi_items * n_slices >= (int64_t)cus * 4 * 4 ||
                                        (CH > 1 && items * n_slices > capacity * 16));
    if (multi) {
        const int64_t per_wg = (multi_items * n_slices + capacity - 1) / capacity;
        WAVES = (int)(per_wg >= 16 ? 16 : (per_wg + 3) / 4 * 4);
    }
    // Fewer items than CUs: a whole workgroup per item, its wavefronts sharing the item's tests.
    constexpr int SPLIT_SEGS = split_lanes(COLS) / COLS;
    const int64_t split_items = (S + SPLIT_SEGS - 1) / SPLIT_SEGS;
    const size_t split_lds = split_lds_bytes(split_lanes(COLS), SPLIT_SEGS, (int)stride);
    const bool split = low_latency && split_items * n_slices <= (int64_t)cus && I >= 2 * CHUNK * SPLIT_WAVES &&
                       split_lds + SPLIT_STATIC_LDS <= (size_t)LDS_SCAN_BYTES &&
                       // the gather addresses W by 24-bit multiplies and a 32-bit byte offset
                       I + np.bias < (1 << 24) && J < (1 << 22) && (I + np.bias) * J * 4 < 0x7fffffffLL;
    if (split) WAVES = 1;                                   // items per workgroup pass
    const int64_t work_items = split ? split_items : multi ? multi_items : items;
    const bool filt = !(split || low_latency);
    if (filt) {
        // the chunk buffers of the wavefronts share the LDS with the slice: fewer wavefronts where it is tight
        // (LDS_SCAN_TARGET leaves room for four)
        while (WAVES > 4 && lds_bytes + filter_extra_lds(COLS, multi ? CH : 1, WAVES) > (size_t)LDS_SCAN_BYTES) WAVES -= 4;
    }
    // split the segments so that slices x groups covers the chip without a second round of workgroups
    int64_t n_groups = capacity / n_slices;
    const int64_t max_groups = (work_items + WAVES - 1) / WAVES;
    if (n_groups > max_groups) n_groups = max_groups;
    if (n_groups < 1) n_groups = 1;
    auto kern_k = filt ? (multi ? scan_filter_kernel<COLS, CH, true> : scan_filter_kernel<COLS, 1, true>)
                  : split ? scan_lds_split_kernel<COLS, true> : scan_lds_kernel<COLS, true>;
    auto kern = filt ? (multi ? scan_filter_kernel<COLS, CH, false> : scan_filter_kernel<COLS, 1, false>)
                : split ? scan_lds_split_kernel<COLS, false> : scan_lds_kernel<COLS, false>;
    dim3 grid((unsigned)(n_slices * n_groups)), block((unsigned)((split && !filt) ? SPLIT_THREADS : WAVES * kWave));
    {
        KernelTimerScope timer_("scan", stream);
        const size_t dyn_lds = filt ? lds_bytes + filter_extra_lds(COLS, multi ? CH : 1, WAVES) : split ? split_lds : lds_bytes;
        if (dyn_lds > (size_t)LDS_SCAN_BYTES)
            return fail(SNNTC_ERR_UNSUPPORTED, "scan: %zu bytes of LDS for %d rows x %d columns exceed the %d available",
                        dyn_lds, (int)(I + np.bias), COLS, LDS_SCAN_BYTES);
        if (causal_k)
            hipLaunchKernelGGL(kern_k, grid, block, dyn_lds, stream, sorted, perm, n_real, w, y, rcp, causal_k,
                               (int)S, (int)I, (int)stride, (int)J, n_slices, (int)n_groups, np, copy);
        else
            hipLaunchKernelGGL(kern, grid, block, dyn_lds, stream, sorted, perm, n_real, w, y, rcp, causal_k,
                               (int)S, (int)I, (int)stride, (int)J, n_slices, (int)n_groups, np, copy);
    }
    SNNTC_HIP_CHECK(hipGetLastError());
    return SNNTC_OK;
}

int launch_scan(const float* sorted, const int32_t* perm, const int32_t* n_real, const float* w, float* y,
                float* rcp, int32_t* causal_k, int64_t S, int64_t I, int64_t stride, int64_t J,
                const NeuronParams& np, const TimeCopy& copy, hipStream_t stream) {
    if (S <= 0 || J <= 0) return SNNTC_OK;
    // widest column slice (8..64) whose I+bias rows fit in LDS; none fits -> stream W from memory
    const size_t rows = (size_t)I + np.bias;
    int cols = 64;
    while (cols > 8 && (rows * cols * sizeof(float) > (size_t)LDS_SCAN_TARGET || cols / 2 >= J)) cols >>= 1;
    const size_t lds_bytes = rows * cols * sizeof(float);
    // (LDS_SCAN_TARGET, not the full 160 KB: whichever LDS kernel the launch shape selects must find room for
    // its chunk buffers behind the slice -- 8-column slices of 5055..5120 rows would fit on their own only)
    if (lds_bytes <= (size_t)LDS_SCAN_TARGET) {
        switch (cols) {
            case 64: return launch_scan_lds<64>(sorted, perm, n_real, w, y, rcp, causal_k, S, I, stride, J, np, copy, lds_bytes, stream);
            case 32: return launch_scan_lds<32>(sorted, perm, n_real, w, y, rcp, causal_k, S, I, stride, J, np, copy, lds_bytes, stream);
            case 16: return launch_scan_lds<16>(sorted, perm, n_real, w, y, rcp, causal_k, S, I, stride, J, np, copy, lds_bytes, stream);
            default: return launch_scan_lds<8>(sorted, perm, n_real, w, y, rcp, causal_k, S, I, stride, J, np, copy, lds_bytes, stream);
        }
    }
    const int j_blocks = (int)((J + kWave - 1) / kWave);
    const int64_t n_items = S * j_blocks;
    const int waves_per_block = 4;
    const int64_t blocks = (n_items + waves_per_block - 1) / waves_per_block;
    if (blocks > 0x7fffffffLL) return fail(SNNTC_ERR_TOO_LARGE, "scan: grid too large");
    dim3 grid((unsigned)blocks), block(waves_per_block * kWave);
    {
        KernelTimerScope timer_("scan_stream", stream);
        if (causal_k)
            hipLaunchKernelGGL(scan_kernel<true>, grid, block, 0, stream, sorted, perm, n_real, w, y, rcp,
                               causal_k, n_items, (int)I, (int)stride, (int)J, j_blocks, np, copy);
        else
            hipLaunchKernelGGL(scan_kernel<false>, grid, block, 0, stream, sorted, perm, n_real, w, y, rcp,
                               causal_k, n_items, (int)I, (int)stride, (int)J, j_blocks, np, copy);
    }
    SNNTC_HIP_CHECK(hipGetLastError());
    return SNNTC_OK;
}

int launch_unpad_rows(const float* sorted, const int32_t* perm, float* sorted_out, int32_t* perm_out,
                      int64_t S, int64_t I, int64_t stride, hipStream_t stream) {
    const int64_t n = S * I;
    if (n <= 0 || (!sorted_out && !perm_out)) return SNNTC_OK;
    {
        KernelTimerScope timer_("unpad_rows", stream);
        hipLaunchKernelGGL(unpad_rows_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, stream, sorted,
                           perm, sorted_out, perm_out, n, (int)I, (int)stride);
    }
    SNNTC_HIP_CHECK(hipGetLastError());
    return SNNTC_OK;
}

}  // namespace snntc
