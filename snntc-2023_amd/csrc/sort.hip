// Segmented stable sort of spike times: one bitonic network per segment, emitting the sorted
// values and the permutation.
//
// Replaces the reference's cub::DeviceSegmentedSort::SortPairs call plus the index-generation and
// im2col temporaries in front of it (snntc/snnfc_kernels.cu.cc:110-155,
// snntc/snncv_kernels.cu.cc:112-166).  Differences by design:
//  * keys are 64-bit composites (order-preserving image of the fp32 value << 32 | source index), so
//    the network -- although not stable by itself -- returns exactly the stable ascending order;
//  * conv patches are gathered straight from the NHWC image, the [B*Nh*Nw, Kh*Kw*C] patch matrix
//    is never written to memory;
//  * a segment is owned by G threads holding EPT consecutive elements each: exchanges at distance
//    < EPT stay in registers, distances below 64 threads use wavefront shuffles, and only
//    segments wider than one wavefront go through LDS.
#include "snntc_common.h"

namespace snntc {
namespace {

typedef unsigned long long u64;

__device__ __forceinline__ uint32_t float_to_key(float f) {
    uint32_t u = __float_as_uint(f);
    if (u == 0x80000000u) u = 0u;                         // -0 sorts together with +0
    return u ^ ((u >> 31) ? 0xffffffffu : 0x80000000u);
}

__device__ __forceinline__ float key_to_float(uint32_t k) {
    return __uint_as_float(k ^ ((k >> 31) ? 0x80000000u : 0xffffffffu));
}

// The value of `v` in lane `lane ^ d`.  Distances 1, 2 and 8 are lane patterns the vector unit applies
// by itself while it moves a register (quad permutes, rotation of a row of 16 by 8); the others go
// through the LDS crossbar, which the four SIMDs of a CU share and which bounds the network otherwise.
__device__ __forceinline__ u64 lane_xor(u64 v, int d) {
    const int lo = (int)(uint32_t)v, hi = (int)(uint32_t)(v >> 32);
    int olo, ohi;
    if (d == 1) {
        olo = __builtin_amdgcn_mov_dpp(lo, 0xB1, 0xf, 0xf, true);      // quad_perm:[1,0,3,2]
        ohi = __builtin_amdgcn_mov_dpp(hi, 0xB1, 0xf, 0xf, true);
    } else if (d == 2) {
        olo = __builtin_amdgcn_mov_dpp(lo, 0x4E, 0xf, 0xf, true);      // quad_perm:[2,3,0,1]
        ohi = __builtin_amdgcn_mov_dpp(hi, 0x4E, 0xf, 0xf, true);
    } else if (d == 8) {
        olo = __builtin_amdgcn_mov_dpp(lo, 0x128, 0xf, 0xf, true);     // row_ror:8
        ohi = __builtin_amdgcn_mov_dpp(hi, 0x128, 0xf, 0xf, true);
    } else {
        return __shfl_xor(v, d, kWave);
    }
    return ((u64)(uint32_t)ohi << 32) | (uint32_t)olo;
}

// RUNS: segments longer than the network are cut into `runs` pieces of NPAD elements; a unit of work is
// one piece, and its sorted keys (value image << 32 | index in the segment; padding keys sort last
// and carry their own position) go to keys[seg][run][NPAD] for the merge passes below.
template <int EPT, int G, int BLOCK, bool RUNS = false>
__global__ void __launch_bounds__(BLOCK)
sort_segments_kernel(SegmentSource src, float* __restrict__ sorted, int32_t* __restrict__ perm,
                     int32_t* __restrict__ n_real, int S, int out_stride, float max_cmp,
                     unsigned long long* __restrict__ keys = nullptr, int runs = 1) {
    constexpr int NPAD = EPT * G;
    constexpr int SEGS = BLOCK / G;
    constexpr bool CROSS_WAVE = G > kWave;
    // the exchange buffer below belongs to the block, not to a segment: a segment that spans several
    // wavefronts must have the block to itself
    static_assert(!CROSS_WAVE || SEGS == 1, "cross-wavefront segments need BLOCK == G");
    __shared__ u64 xchg[CROSS_WAVE ? NPAD : 1];
    __shared__ int wave_count[CROSS_WAVE ? G / kWave : 1];

    const int tseg = threadIdx.x % G;
    int seg = blockIdx.x * SEGS + threadIdx.x / G;
    int e0 = 0;                                           // first element of the unit in its segment
    if constexpr (RUNS) {
        const int unit = seg;
        seg = unit / runs;
        e0 = (unit - seg * runs) * NPAD;
    }
    const bool live = seg < S;
    const int I = src.I;

    // ---- load EPT consecutive elements, pad with keys that sort after every real value --------
    u64 v[EPT];
    {
        const float* p = src.base;
        int kh = 0, rem = 0, row = 0, span = 1;
        if (live) {
            if (src.conv) {
                const int per_img = src.Nh * src.Nw;
                const int a = seg / per_img, r2 = seg - a * per_img;
                const int nh = r2 / src.Nw, nw = r2 - nh * src.Nw;
                p += ((size_t)(a * src.H + nh * src.Sh) * src.W + (size_t)nw * src.Sw) * src.C;
                span = src.Kw * src.C;          // contiguous floats per kernel row
                row = src.W * src.C;            // floats per image row
                kh = (e0 + tseg * EPT) / span;
                rem = e0 + tseg * EPT - kh * span;
            } else {
                p += (size_t)seg * I;
            }
        }
#pragma unroll
        for (int r = 0; r < EPT; ++r) {
            const int e = e0 + tseg * EPT + r;
            uint32_t key = 0xffffffffu;
            if (live && e < I) {
                float f;
                if (src.conv) {
                    f = p[(size_t)kh * row + rem];
                    if (++rem == span) { rem = 0; ++kh; }
                } else {
                    f = p[e];
                }
                key = float_to_key(f);
            }
            v[r] = ((u64)key << 32) | (uint32_t)e;
        }
    }

    // ---- bitonic network ------------------------------------------------------------------------
#pragma unroll
    for (int k = 2; k <= NPAD; k <<= 1) {
        // partners in other threads: element distance j >= EPT
#pragma unroll
        for (int j = k >> 1; j >= EPT; j >>= 1) {
            const int d = j / EPT;
            const bool lower = (tseg & d) == 0;
            const bool up = ((tseg * EPT) & k) == 0;
            const bool keep_min = (lower == up);
            if (CROSS_WAVE && d >= kWave) {
                __syncthreads();
#pragma unroll
                for (int r = 0; r < EPT; ++r) xchg[r * G + tseg] = v[r];
                __syncthreads();
#pragma unroll
                for (int r = 0; r < EPT; ++r) {
                    const u64 o = xchg[r * G + (tseg ^ d)];
                    const bool take = (o < v[r]) == keep_min;
                    v[r] = take ? o : v[r];
                }
            } else {
#pragma unroll
                for (int r = 0; r < EPT; ++r) {
                    const u64 o = lane_xor(v[r], d);
                    const bool take = (o < v[r]) == keep_min;
                    v[r] = take ? o : v[r];
                }
            }
        }
        // partners inside the thread: element distance j < EPT
#pragma unroll
        for (int j = (EPT >> 1); j >= 1; j >>= 1) {
            if (j <= (k >> 1)) {
#pragma unroll
                for (int r = 0; r < EPT; ++r) {
                    if ((r & j) == 0) {
                        const bool up = ((tseg * EPT + r) & k) == 0;
                        const u64 a = v[r], b = v[r | j];
                        const bool sw = (a > b) == up;
                        v[r] = sw ? b : a;
                        v[r | j] = sw ? a : b;
                    }
                }
            }
        }
    }

    if constexpr (RUNS) {
        if (live) {
            u64* ko = keys + ((size_t)seg * runs) * NPAD + e0 + tseg * EPT;
#pragma unroll
            for (int r = 0; r < EPT; ++r) ko[r] = v[r];
        }
        return;
    }
    // ---- store: rows are out_stride long; positions past the segment get (+inf, row 0) ------------
    int below = 0;                      // own elements that take part in the scan (value <= MAX-0.1)
    // (out_stride is a multiple of 16 and EPT divides 16: a thread's EPT positions lie inside the row
    // or outside it as a whole, and its part of the row is stored as 8- or 16-byte pieces)
    if (live && tseg * EPT < out_stride) {
        float fo[EPT];
        int32_t io[EPT];
#pragma unroll
        for (int r = 0; r < EPT; ++r) {
            const bool real = tseg * EPT + r < I;
            const float f = key_to_float((uint32_t)(v[r] >> 32));
            fo[r] = real ? f : INFINITY;
            io[r] = real ? (int32_t)(uint32_t)v[r] : 0;
            below += (real && f <= max_cmp) ? 1 : 0;
        }
        float* so = sorted + (size_t)seg * out_stride + tseg * EPT;
        int32_t* po = perm + (size_t)seg * out_stride + tseg * EPT;
        if constexpr (EPT == 2) {
            *reinterpret_cast<float2*>(so) = make_float2(fo[0], fo[1]);
            *reinterpret_cast<int2*>(po) = make_int2(io[0], io[1]);
        } else {
#pragma unroll
            for (int r = 0; r < EPT; r += 4) {
                *reinterpret_cast<float4*>(so + r) = make_float4(fo[r], fo[r + 1], fo[r + 2], fo[r + 3]);
                *reinterpret_cast<int4*>(po + r) = make_int4(io[r], io[r + 1], io[r + 2], io[r + 3]);
            }
        }
    }
    // ---- number of scan inputs per segment: sum of `below` over the segment's G threads -----------
    if (n_real != nullptr) {
#pragma unroll
        for (int d = 1; d < (G < kWave ? G : kWave); d <<= 1) below += __shfl_xor(below, d, kWave);
        if (CROSS_WAVE) {
            if ((threadIdx.x % kWave) == 0) wave_count[threadIdx.x / kWave] = below;
            __syncthreads();
            if (threadIdx.x == 0) {
                int total = 0;
                for (int wv = 0; wv < G / kWave; ++wv) total += wave_count[wv];
                n_real[seg] = total;
            }
        } else if (live && tseg == 0) {
            n_real[seg] = below;
        }
    }
}

template <int EPT, int G>
int launch_sort_t(const SegmentSource& src, int64_t S, float* sorted, int32_t* perm, int32_t* n_real,
                  int out_stride, float max_cmp, hipStream_t stream) {
    constexpr int BLOCK = G > 256 ? G : 256;
    constexpr int SEGS = BLOCK / G;
    const int64_t blocks = (S + SEGS - 1) / SEGS;
    if (blocks > 0x7fffffffLL) return fail(SNNTC_ERR_TOO_LARGE, "sort: too many segments (%lld)", (long long)S);
    { KernelTimerScope timer_("sort_segments", stream);
    hipLaunchKernelGGL((sort_segments_kernel<EPT, G, BLOCK>), dim3((unsigned)blocks), dim3(BLOCK), 0, stream,
                       src, sorted, perm, n_real, (int)S, out_stride, max_cmp);
    }
    SNNTC_HIP_CHECK(hipGetLastError());
    return SNNTC_OK;
}

// ---------------------------------------------------------------------------------------------
// Segments longer than the largest network (kMaxSegment): the pieces sorted by the RUNS
// instantiation above are merged pairwise, pass after pass, in global memory.  A wavefront
// produces MERGE_TILE consecutive keys of a merged pair: every lane finds by binary search how
// many of the keys before its share come from the first run (merge path) and then merges its
// share step by step.  Keys are distinct (they contain the index), so the result is the stable
// order whatever the pass structure.  The last pass writes the (value, index) rows the scan reads,
// with (+inf, 0) past the segment's end.  Rare and long: written for simplicity, not for speed.
// ---------------------------------------------------------------------------------------------
constexpr int MERGE_TILE = 1024;
constexpr int MERGE_PER_LANE = MERGE_TILE / kWave;

__global__ void __launch_bounds__(256)
merge_runs_kernel(const u64* __restrict__ in, u64* __restrict__ out, float* __restrict__ sorted,
                  int32_t* __restrict__ perm, int S, int I, int total, int L, int out_stride, int last) {
    const int lane = threadIdx.x % kWave;
    const int64_t tile = (int64_t)blockIdx.x * (blockDim.x / kWave) + threadIdx.x / kWave;
    const int tiles_per_seg = total / MERGE_TILE;
    const int seg = (int)(tile / tiles_per_seg);
    if (seg >= S) return;
    const int pos0 = (int)(tile - (int64_t)seg * tiles_per_seg) * MERGE_TILE;       // first output of the tile
    const int base = pos0 / (2 * L) * (2 * L);                                      // first key of the pair
    const int nA = min(L, total - base), nB = min(L, max(0, total - base - L));
    const u64* A = in + (size_t)seg * total + base;
    const u64* B = A + L;
    const int d0 = pos0 - base + lane * MERGE_PER_LANE;
    int lo = max(0, d0 - nB), hi = min(d0, nA);
    while (lo < hi) {
        const int mid = (lo + hi) >> 1;
        if (A[mid] < B[d0 - mid - 1]) lo = mid + 1; else hi = mid;                 // A[mid] precedes B[j-1]: too few from A
    }
    int i = lo, j = d0 - lo;
    for (int u = 0; u < MERGE_PER_LANE; ++u) {
        const u64 a = i < nA ? A[i] : ~0ull, b = j < nB ? B[j] : ~0ull;
        const bool take_a = a < b;
        const u64 key = take_a ? a : b;
        i += take_a ? 1 : 0;
        j += take_a ? 0 : 1;
        const int q = base + d0 + u;
        if (!last) {
            out[(size_t)seg * total + q] = key;
        } else if (q < I) {
            sorted[(size_t)seg * out_stride + q] = key_to_float((uint32_t)(key >> 32));
            perm[(size_t)seg * out_stride + q] = (int32_t)(uint32_t)key;
        } else if (q < out_stride) {
            sorted[(size_t)seg * out_stride + q] = INFINITY;
            perm[(size_t)seg * out_stride + q] = 0;
        }
    }
}

// n_real[seg] = entries of the sorted row that take part in the scan (value <= max_cmp)
__global__ void __launch_bounds__(256)
count_real_kernel(const float* __restrict__ sorted, int32_t* __restrict__ n_real, int I, int out_stride, float max_cmp) {
    __shared__ int part[256 / kWave];
    const float* row = sorted + (size_t)blockIdx.x * out_stride;
    int n = 0;
    for (int e = threadIdx.x; e < I; e += blockDim.x) n += row[e] <= max_cmp ? 1 : 0;
#pragma unroll
    for (int d = 1; d < kWave; d <<= 1) n += __shfl_xor(n, d, kWave);
    if (threadIdx.x % kWave == 0) part[threadIdx.x / kWave] = n;
    __syncthreads();
    if (threadIdx.x == 0) n_real[blockIdx.x] = part[0] + part[1] + part[2] + part[3];
}

int launch_sort_long(const SegmentSource& src, int64_t S, float* sorted, int32_t* perm, int32_t* n_real,
                     int out_stride, float max_cmp, void* long_ws, hipStream_t stream) {
    if (!long_ws) return fail(SNNTC_ERR_WORKSPACE, "sort: segments of %d inputs need the long-segment workspace", src.I);
    const int runs = (src.I + kMaxSegment - 1) / kMaxSegment;
    const int64_t total = (int64_t)runs * kMaxSegment;
    if (S * total > 0x7fffffffLL * 8) return fail(SNNTC_ERR_TOO_LARGE, "sort: %lld segments of %d inputs", (long long)S, src.I);
    u64* buf[2] = {static_cast<u64*>(long_ws), static_cast<u64*>(long_ws) + S * total};
    if (S * runs > 0x7fffffffLL) return fail(SNNTC_ERR_TOO_LARGE, "sort: too many segments (%lld)", (long long)S);
    KernelTimerScope timer_("sort_segments", stream);
    hipLaunchKernelGGL((sort_segments_kernel<8, 1024, 1024, true>), dim3((unsigned)(S * runs)), dim3(1024), 0, stream, src,
                       sorted, perm, nullptr, (int)S, out_stride, max_cmp, buf[0], runs);
    const int64_t tiles = S * (total / MERGE_TILE);
    const int64_t blocks = (tiles + 3) / 4;
    if (blocks > 0x7fffffffLL) return fail(SNNTC_ERR_TOO_LARGE, "sort: grid too large");
    int cur = 0;
    for (int64_t L = kMaxSegment; L < total; L *= 2) {
        const int last = 2 * L >= total;
        hipLaunchKernelGGL(merge_runs_kernel, dim3((unsigned)blocks), dim3(256), 0, stream, buf[cur], buf[cur ^ 1], sorted,
                           perm, (int)S, src.I, (int)total, (int)L, out_stride, last);
        cur ^= 1;
    }
    if (n_real)
        hipLaunchKernelGGL(count_real_kernel, dim3((unsigned)S), dim3(256), 0, stream, sorted, n_real, src.I, out_stride,
                           max_cmp);
    SNNTC_HIP_CHECK(hipGetLastError());
    return SNNTC_OK;
}

}  // namespace

// Bytes of the extra workspace launch_sort needs for S segments of I inputs (0 up to kMaxSegment):
// two key buffers for the merge passes.
size_t sort_long_workspace_bytes(int64_t S, int64_t I) {
    if (I <= kMaxSegment) return 0;
    const int64_t runs = (I + kMaxSegment - 1) / kMaxSegment;
    return (size_t)2 * S * runs * kMaxSegment * sizeof(u64);
}

int launch_sort(const SegmentSource& src, int64_t S, float* sorted, int32_t* perm, int32_t* n_real,
                int out_stride, float max_cmp, void* long_ws, hipStream_t stream) {
    if (S <= 0 || src.I <= 0) return SNNTC_OK;
    const int I = src.I;
    if (I > kMaxSegment) return launch_sort_long(src, S, sorted, perm, n_real, out_stride, max_cmp, long_ws, stream);
    if (I <= 32)   return launch_sort_t<2, 16>(src, S, sorted, perm, n_real, out_stride, max_cmp, stream);
    if (I <= 64)   return launch_sort_t<2, 32>(src, S, sorted, perm, n_real, out_stride, max_cmp, stream);
    if (I <= 128)  return launch_sort_t<2, 64>(src, S, sorted, perm, n_real, out_stride, max_cmp, stream);
    // many segments of 129..256 (the patches of a 7x7x3 stem): two segments per wavefront, eight
    // elements per thread -- five of the network's steps stay inside a thread instead of three
    // (401408 segments of 147: 417 us against 465 us)
    if (I <= 256 && I > 128 && S >= 65536) return launch_sort_t<8, 32>(src, S, sorted, perm, n_real, out_stride, max_cmp, stream);
    if (I <= 256)  return launch_sort_t<4, 64>(src, S, sorted, perm, n_real, out_stride, max_cmp, stream);
    // Few long segments (a dense batch): several wavefronts per segment with two or four elements per
    // thread instead of one wavefront with eight or more -- the chip fills, and a lone wavefront's long
    // network is what such a launch waits for.  Rows of 257..512: 7 against 12 us up to 512 rows, the
    // same from 2048 rows on; rows of 513..1024: 29 against 58 us at 2048 rows, 148 against 183 us at
    // 16384, so at every count; rows of 1025..2048: 12 against 15 us up to 128 rows, behind from 8192 on.
    if (I <= 512 && S <= 2048) return launch_sort_t<2, 256>(src, S, sorted, perm, n_real, out_stride, max_cmp, stream);
    if (I <= 512)  return launch_sort_t<8, 64>(src, S, sorted, perm, n_real, out_stride, max_cmp, stream);
    if (I <= 1024) return launch_sort_t<2, 512>(src, S, sorted, perm, n_real, out_stride, max_cmp, stream);
    if (I <= 2048 && S <= 512) return launch_sort_t<4, 512>(src, S, sorted, perm, n_real, out_stride, max_cmp, stream);
    if (I <= 2048) return launch_sort_t<8, 256>(src, S, sorted, perm, n_real, out_stride, max_cmp, stream);
    if (I <= 4096) return launch_sort_t<8, 512>(src, S, sorted, perm, n_real, out_stride, max_cmp, stream);
    return launch_sort_t<8, 1024>(src, S, sorted, perm, n_real, out_stride, max_cmp, stream);
}

}  // namespace snntc
