// Patch sort for conv layers by merging pre-sorted pixels.
//
// A conv patch is Kh*Kw pixels of C channels; neighbouring patches share most of their pixels, so
// sorting every patch from scratch repeats the same comparisons Kh*Kw times.  Here every pixel of
// the padded image is sorted once (sort_segments_kernel on [B*H*W, C] rows), and a patch is put
// together by rank computation instead of a sorting network:
//   1. column lists: the Kh pixels of one image column under the window merge into a list of
//      Kh*C elements; rank = own position + (elements of the other pixels that precede it),
//      each count one binary search.  A column list serves every patch of the tile that covers it.
//   2. patch: the Kw column lists merge the same way into the P = Kh*Kw*C sorted entries.
// "Precedes" is the stable order of the flat patch index (kh, kw, c): smaller value first, equal
// values by (kh, kw, c).  Column lists carry 64-bit keys  orderable(value) << 32 | kh << 16 | c,
// so one unsigned compare against a threshold decides precedence including ties.
// The result is identical to the bitonic path (and to a stable argsort); it replaces the same
// reference code (snntc/snncv_kernels.cu.cc:112-166).
#include <atomic>

#include "snntc_common.h"

namespace snntc {
namespace {

typedef unsigned long long u64;

__device__ __forceinline__ uint32_t order_key(float f) {
    uint32_t u = __float_as_uint(f);
    if (u == 0x80000000u) u = 0u;                         // -0 sorts together with +0
    return u ^ ((u >> 31) ? 0xffffffffu : 0x80000000u);
}

__device__ __forceinline__ float order_key_to_float(uint32_t k) {
    return __uint_as_float(k ^ ((k >> 31) ? 0x80000000u : 0xffffffffu));
}

// Batched binary searches.  One search is a chain of dependent LDS reads; a lane therefore runs
// NB of them side by side (different elements against the same list) so their reads overlap.
constexpr int NB = 4;

// cnt[i] += number of entries of the ascending list[0..n) that precede a[i]: entries < a[i] when
// strict, <= a[i] otherwise.
template <bool STRICT>
__device__ __forceinline__ void count_before_f32(const float* list, int n, const float (&a)[NB], int (&cnt)[NB]) {
    int base[NB];
#pragma unroll
    for (int i = 0; i < NB; ++i) base[i] = 0;
    int len = n;
    while (len > 1) {
        const int half = len >> 1;
        float v[NB];
#pragma unroll
        for (int i = 0; i < NB; ++i) v[i] = list[base[i] + half - 1];
#pragma unroll
        for (int i = 0; i < NB; ++i) base[i] += (STRICT ? (v[i] < a[i]) : (v[i] <= a[i])) ? half : 0;
        len -= half;
    }
#pragma unroll
    for (int i = 0; i < NB; ++i) {
        const float v = list[base[i]];
        cnt[i] += base[i] + ((STRICT ? (v < a[i]) : (v <= a[i])) ? 1 : 0);
    }
}

// cnt[i] += (entries of key list A that are < thrA[i]) + (entries of key list B that are < thrB[i]);
// both lists ascending with n entries.  2*EB chains run side by side.
template <int EB>
__device__ __forceinline__ void count_below_u64_pair(const u64* listA, const u64* listB, int n,
                                                     const u64 (&thrA)[EB], const u64 (&thrB)[EB], int (&cnt)[EB]) {
    int ba[EB], bb[EB];
#pragma unroll
    for (int i = 0; i < EB; ++i) { ba[i] = 0; bb[i] = 0; }
    int len = n;
    while (len > 1) {
        const int half = len >> 1;
        u64 va[EB], vb[EB];
#pragma unroll
        for (int i = 0; i < EB; ++i) { va[i] = listA[ba[i] + half - 1]; vb[i] = listB[bb[i] + half - 1]; }
#pragma unroll
        for (int i = 0; i < EB; ++i) {
            ba[i] += va[i] < thrA[i] ? half : 0;
            bb[i] += vb[i] < thrB[i] ? half : 0;
        }
        len -= half;
    }
#pragma unroll
    for (int i = 0; i < EB; ++i)
        cnt[i] += ba[i] + (listA[ba[i]] < thrA[i] ? 1 : 0) + bb[i] + (listB[bb[i]] < thrB[i] ? 1 : 0);
}

template <int EB>
__device__ __forceinline__ void count_below_u64(const u64* list, int n, const u64 (&thr)[EB], int (&cnt)[EB]) {
    int base[EB];
#pragma unroll
    for (int i = 0; i < EB; ++i) base[i] = 0;
    int len = n;
    while (len > 1) {
        const int half = len >> 1;
        u64 v[EB];
#pragma unroll
        for (int i = 0; i < EB; ++i) v[i] = list[base[i] + half - 1];
#pragma unroll
        for (int i = 0; i < EB; ++i) base[i] += v[i] < thr[i] ? half : 0;
        len -= half;
    }
#pragma unroll
    for (int i = 0; i < EB; ++i) cnt[i] += base[i] + (list[base[i]] < thr[i] ? 1 : 0);
}

constexpr int MERGE_THREADS = 256;
constexpr int MERGE_WAVES = MERGE_THREADS / kWave;

// One workgroup = TW consecutive patches of one output row.
//   pix_z / pix_c : every pixel's channels sorted ascending and their channel ids, rows of Cs entries
//   sorted / perm : [S, stride] outputs (entries past P padded with +inf / 0), n_real[S]
template <int EB>   // own-column elements a lane ranks per pass
__global__ void __launch_bounds__(MERGE_THREADS)
merge_patches_kernel(const float* __restrict__ pix_z, const int32_t* __restrict__ pix_c, int Cs,
                     float* __restrict__ sorted, int32_t* __restrict__ perm, int32_t* __restrict__ n_real,
                     int H, int W, int C, int Kh, int Kw, int Sh, int Sw, int Nh, int Nw, int TW, int tiles_w,
                     int stride, float max_cmp) {
    extern __shared__ __align__(16) unsigned char lds_raw[];
    const int tile_cols = (TW - 1) * Sw + Kw;
    const int KhC = Kh * C;
    const int P = KhC * Kw;
    // LDS carve-up (8-byte pieces first)
    // The pixel lists are dead once the column lists exist; the per-wave output staging reuses
    // their space.
    u64* col_keys = reinterpret_cast<u64*>(lds_raw);                                   // [tile_cols][KhC]
    u64* out_keys = col_keys + (size_t)tile_cols * KhC;                                // [MERGE_WAVES][P]
    float* px_z = reinterpret_cast<float*>(out_keys);                                  // [Kh][tile_cols][C]
    uint16_t* px_c = reinterpret_cast<uint16_t*>(px_z + (size_t)Kh * tile_cols * C);   // [Kh][tile_cols][C]

    const int tile = blockIdx.x % tiles_w;
    const int rowid = blockIdx.x / tiles_w;
    const int nh = rowid % Nh, a = rowid / Nh;
    const int nw0 = tile * TW;
    const int w_first = nw0 * Sw;

    // ---- stage the sorted pixels under the tile ------------------------------------------------
    const int n_px = Kh * tile_cols * C;
    // loads are issued in batches: one at a time would cost a memory latency per element
    constexpr int STAGE = 8;
    for (int base = threadIdx.x; base < n_px; base += STAGE * MERGE_THREADS) {
        float zv[STAGE];
        int cv[STAGE];
#pragma unroll
        for (int u = 0; u < STAGE; ++u) {
            const int idx = base + u * MERGE_THREADS;
            const int c = idx % C;
            const int pc = idx / C;
            const int col = pc % tile_cols, kh = pc / tile_cols;
            const int wp = w_first + col;
            zv[u] = INFINITY;
            cv[u] = c;
            if (idx < n_px && wp < W) {
                const size_t g = ((size_t)(a * H + nh * Sh + kh) * W + wp) * Cs + c;
                zv[u] = pix_z[g];
                cv[u] = pix_c[g];
            }
        }
#pragma unroll
        for (int u = 0; u < STAGE; ++u) {
            const int idx = base + u * MERGE_THREADS;
            if (idx < n_px) { px_z[idx] = zv[u]; px_c[idx] = (uint16_t)cv[u]; }
        }
    }
    __syncthreads();

    // ---- column lists: merge the Kh pixels of every column -----------------------------------------
    // A thread takes NB elements of the same (kh, col) pixel list at a time (idx, idx+1, ...).
    for (int idx0 = threadIdx.x * NB; idx0 < n_px; idx0 += MERGE_THREADS * NB) {
        // C is a multiple of NB, so the NB elements share their pixel
        const int l0 = idx0 % C;
        const int pc = idx0 / C;
        const int col = pc % tile_cols, kh = pc / tile_cols;
        float z[NB];
        int rank[NB];
#pragma unroll
        for (int i = 0; i < NB; ++i) { z[i] = px_z[idx0 + i]; rank[i] = l0 + i; }
        for (int k2 = 0; k2 < kh; ++k2)          // pixels above: equal values come first there
            count_before_f32<false>(px_z + (size_t)(k2 * tile_cols + col) * C, C, z, rank);
        for (int k2 = kh + 1; k2 < Kh; ++k2)     // pixels below: only strictly smaller values precede
            count_before_f32<true>(px_z + (size_t)(k2 * tile_cols + col) * C, C, z, rank);
#pragma unroll
        for (int i = 0; i < NB; ++i)
            col_keys[(size_t)col * KhC + rank[i]] =
                ((u64)order_key(z[i]) << 32) | ((u64)kh << 16) | px_c[idx0 + i];
    }
    __syncthreads();

    // ---- patches: merge the Kw columns of every patch ----------------------------------------------
    const int lane = threadIdx.x % kWave;
    const int wave = threadIdx.x / kWave;
    u64* my_out = out_keys + (size_t)wave * P;
    const int rounds = (TW + MERGE_WAVES - 1) / MERGE_WAVES;
    for (int rd = 0; rd < rounds; ++rd) {
        const int j = rd * MERGE_WAVES + wave;
        const bool valid = j < TW && nw0 + j < Nw;
        if (valid) {
            for (int kw = 0; kw < Kw; ++kw) {
                const u64* mine = col_keys + (size_t)(j * Sw + kw) * KhC;
                // EB elements of the own column per pass (lane, lane+64, ...); a tail element repeats
                // the last one and is not written.  The other columns are taken two at a time.
                for (int e0 = lane; e0 < KhC; e0 += kWave * EB) {
                    u64 key[EB], thr_incl[EB], thr_strict[EB];
                    int rank[EB];
#pragma unroll
                    for (int i = 0; i < EB; ++i) {
                        const int e = min(e0 + i * kWave, KhC - 1);
                        key[i] = mine[e];
                        const u64 hi = key[i] & 0xffffffff00000000ull;
                        const u64 kh = (key[i] >> 16) & 0xffffull;
                        // entries of a column to the left precede on (value, kh) <= mine, to the right on <
                        thr_incl[i] = hi | ((kh + 1) << 16);
                        thr_strict[i] = hi | (kh << 16);
                        rank[i] = e;
                    }
                    const u64* cols = col_keys + (size_t)(j * Sw) * KhC;
                    int k2 = 0;
                    for (; k2 + 1 < kw; k2 += 2)             // two columns to the left
                        count_below_u64_pair<EB>(cols + (size_t)k2 * KhC, cols + (size_t)(k2 + 1) * KhC, KhC,
                                                 thr_incl, thr_incl, rank);
                    int k3 = kw + 1;
                    if (k2 < kw && k3 < Kw) {                // one left, one right
                        count_below_u64_pair<EB>(cols + (size_t)k2 * KhC, cols + (size_t)k3 * KhC, KhC, thr_incl,
                                                 thr_strict, rank);
                        ++k2; ++k3;
                    }
                    if (k2 < kw) count_below_u64<EB>(cols + (size_t)k2 * KhC, KhC, thr_incl, rank);
                    for (; k3 + 1 < Kw; k3 += 2)             // two columns to the right
                        count_below_u64_pair<EB>(cols + (size_t)k3 * KhC, cols + (size_t)(k3 + 1) * KhC, KhC,
                                                 thr_strict, thr_strict, rank);
                    if (k3 < Kw) count_below_u64<EB>(cols + (size_t)k3 * KhC, KhC, thr_strict, rank);
#pragma unroll
                    for (int i = 0; i < EB; ++i) {
                        if (e0 + i * kWave < KhC) {
                            const uint32_t kh = (uint32_t)(key[i] >> 16) & 0xffffu, c = (uint32_t)key[i] & 0xffffu;
                            my_out[rank[i]] = (key[i] & 0xffffffff00000000ull) | (u64)((kh * Kw + kw) * C + c);
                        }
                    }
                }
            }
        }
        __syncthreads();
        if (valid) {
            const size_t s = (size_t)(a * Nh + nh) * Nw + nw0 + j;
            float* so = sorted + s * stride;
            int32_t* po = perm + s * stride;
            int below = 0;
            for (int e = lane; e < stride; e += kWave) {
                float z = INFINITY;
                int32_t id = 0;
                if (e < P) {
                    const u64 key = my_out[e];
                    z = order_key_to_float((uint32_t)(key >> 32));
                    id = (int32_t)(uint32_t)key;
                    below += z <= max_cmp ? 1 : 0;
                }
                so[e] = z;
                po[e] = id;
            }
#pragma unroll
            for (int d = 1; d < kWave; d <<= 1) below += __shfl_xor(below, d, kWave);
            if (lane == 0) n_real[s] = below;
        }
        __syncthreads();
    }
}

size_t merge_lds_bytes(int C, int Kh, int Kw, int Sw, int TW) {
    const size_t tile_cols = (size_t)(TW - 1) * Sw + Kw;
    const size_t KhC = (size_t)Kh * C, P = KhC * Kw;
    const size_t staging = (size_t)MERGE_WAVES * P * 8, pixels = (size_t)Kh * tile_cols * C * (4 + 2);
    return tile_cols * KhC * 8 + (staging > pixels ? staging : pixels);
}

// Patches per tile: as many as fit in 52 KB of LDS (so three workgroups share a CU), at
// most 16, never more than the row holds.  Layers with so many channels that not even two
// patches fit in 52 KB take what fits in MERGE_LDS_CAP (one workgroup per CU).
constexpr size_t MERGE_LDS_CAP = 128 * 1024;
int merge_tile_width(const ConvGeom& g) {
    const int tw_max = g.Nw < 16 ? (int)g.Nw : 16;
    int tw = tw_max;
    while (tw > 1 && merge_lds_bytes((int)g.C, (int)g.Kh, (int)g.Kw, (int)g.Sw, tw) > 52 * 1024) --tw;
    if (tw < 2) {
        tw = tw_max;
        while (tw > 1 && merge_lds_bytes((int)g.C, (int)g.Kh, (int)g.Kw, (int)g.Sw, tw) > MERGE_LDS_CAP) --tw;
    }
    return tw;
}

}  // namespace

// The merge path needs channel ids and kh in 16 bits, a useful amount of sharing and an LDS
// footprint within reach; everything else goes through the bitonic network.
bool merge_sort_supported(const ConvGeom& g) {
    if (g.C < 32 || g.C % NB != 0 || g.C > 4096 || g.Kh * g.Kw < 2 || g.Kh > 255) return false;
    const int tw = merge_tile_width(g);
    return merge_lds_bytes((int)g.C, (int)g.Kh, (int)g.Kw, (int)g.Sw, tw) <= MERGE_LDS_CAP && tw >= 2;
}

// One-time set-up on device `dev` (the current device): the dynamic-LDS limit of every
// instantiation, so that no later launch calls hipFuncSetAttribute (not allowed during capture).
int merge_prepare_device(int dev) {
    static std::atomic<bool> done[kMaxDevices];
    if (dev < 0 || dev >= kMaxDevices) return fail(SNNTC_ERR_UNSUPPORTED, "patch merge: device index %d not supported", dev);
    if (done[dev].load(std::memory_order_acquire)) return SNNTC_OK;
    const void* kernels[] = {reinterpret_cast<const void*>(merge_patches_kernel<1>),
                             reinterpret_cast<const void*>(merge_patches_kernel<2>),
                             reinterpret_cast<const void*>(merge_patches_kernel<3>),
                             reinterpret_cast<const void*>(merge_patches_kernel<4>)};
    for (const void* k : kernels)
        SNNTC_HIP_CHECK(hipFuncSetAttribute(k, hipFuncAttributeMaxDynamicSharedMemorySize, (int)MERGE_LDS_CAP));
    done[dev].store(true, std::memory_order_release);
    return SNNTC_OK;
}

int launch_merge_patches(const float* pix_z, const int32_t* pix_c, int64_t Cs, float* sorted, int32_t* perm,
                         int32_t* n_real, const ConvGeom& g, int64_t stride, float max_cmp,
                         hipStream_t stream) {
    const int tw = merge_tile_width(g);
    const size_t lds = merge_lds_bytes((int)g.C, (int)g.Kh, (int)g.Kw, (int)g.Sw, tw);
    const int tiles_w = (int)((g.Nw + tw - 1) / tw);
    const int64_t blocks = g.B * g.Nh * tiles_w;
    if (blocks > 0x7fffffffLL) return fail(SNNTC_ERR_TOO_LARGE, "patch merge: grid too large");
    // elements of one column per lane: Kh*C / 64, at most four ranked side by side
    const int64_t per_lane = (g.Kh * g.C + kWave - 1) / kWave;
    const int eb = per_lane >= 4 ? 4 : (int)per_lane;
    auto kern = eb == 1 ? merge_patches_kernel<1> : eb == 2 ? merge_patches_kernel<2>
              : eb == 3 ? merge_patches_kernel<3> : merge_patches_kernel<4>;
    int dev = 0;
    SNNTC_HIP_CHECK(hipGetDevice(&dev));
    const int prep = merge_prepare_device(dev);
    if (prep) return prep;
    {
        KernelTimerScope timer_("merge_patches", stream);
        hipLaunchKernelGGL(kern, dim3((unsigned)blocks), dim3(MERGE_THREADS), lds, stream, pix_z, pix_c, (int)Cs,
                           sorted, perm, n_real, (int)g.H, (int)g.W, (int)g.C, (int)g.Kh, (int)g.Kw, (int)g.Sh,
                           (int)g.Sw, (int)g.Nh, (int)g.Nw, tw, tiles_w, (int)stride, max_cmp);
    }
    SNNTC_HIP_CHECK(hipGetLastError());
    return SNNTC_OK;
}

}  // namespace snntc
