// Patch sort for conv layers by merging pre-sorted pixels.
//
// A conv patch is Kh*Kw pixels of C channels; neighbouring patches share most of their pixels, so
// sorting every patch from scratch repeats the same comparisons Kh*Kw times.  Here every pixel of
// the padded image is sorted once (sort_segments_kernel on [B*H*W, C] rows), and a patch is put
// together by rank computation instead of a sorting network:
//   1. column lists: the Kh pixels of one image column under the window merge into a list of
//      Kh*C elements; rank = own position + (elements of the other pixels that precede it),
//      each count one binary search.  A column list serves every patch of the tile that covers it.
//   2. patch: the Kw column lists are merged one after the other (list 0 with 1, the result with 2,
//      ...) by a wavefront; every lane takes a run of consecutive outputs, finds where its run starts
//      in the two inputs with one binary search (merge path) and then merges sequentially.
// "Precedes" is the stable order of the flat patch index (kh, kw, c): smaller value first, equal
// values by (kh, kw, c).  Column lists carry 64-bit keys  orderable(value) << 32 | kh << 24 | c with
// an empty field for kw at bit 16, which a patch fills in as it reads a column; all keys of a patch
// are then distinct and one unsigned compare decides precedence including ties.
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

// Merges the ascending key lists A[0..nA) and B[0..nB) (all keys distinct once `orB` is or-ed into
// the keys of B and those of A have become (a | orA) - subA; both lists are followed by an all-ones
// sentinel, which stays above every key under these changes) into out[0..nA+nB), with one
// wavefront, and ends `out` with a sentinel of its own.  A lane produces RUNS runs of E consecutive
// outputs each (independent chains of LDS reads that overlap): a binary search along the diagonal
// i + j = first output finds how many of a run's outputs come from A, then one output per step.  `out` must not overlap the inputs (the lanes of a wavefront read and write side by side).
template <int RUNS>
__device__ __forceinline__ void wave_merge(const u64* A, int nA, const u64* B, int nB, u64 orB, u64* out, int lane,
                                           u64 orA = 0, u64 subA = 0) {
    const int n = nA + nB;
    const int E = (n + kWave * RUNS - 1) / (kWave * RUNS);
    int d0[RUNS], d1[RUNS], lo[RUNS], hi[RUNS];
#pragma unroll
    for (int r = 0; r < RUNS; ++r) {
        d0[r] = min((lane * RUNS + r) * E, n);
        d1[r] = min(d0[r] + E, n);
        lo[r] = max(0, d0[r] - nB);
        hi[r] = min(d0[r], nA);
    }
    const int iters = 32 - __builtin_clz(min(nA, nB) | 1);            // wave-uniform bound on the search length
    for (int it = 0; it < iters; ++it) {
        u64 a[RUNS], b[RUNS];
        int mid[RUNS];
#pragma unroll
        for (int r = 0; r < RUNS; ++r) {
            mid[r] = (lo[r] + hi[r]) >> 1;
            const bool open = lo[r] < hi[r];
            a[r] = A[open ? mid[r] : 0];
            b[r] = B[open ? d0[r] - mid[r] - 1 : 0];
        }
#pragma unroll
        for (int r = 0; r < RUNS; ++r) {
            const bool open = lo[r] < hi[r];
            const bool a_first = ((a[r] | orA) - subA) < (b[r] | orB); // A[i] goes before B[j-1]: i is too small
            lo[r] = (open && a_first) ? mid[r] + 1 : lo[r];
            hi[r] = (open && !a_first) ? mid[r] : hi[r];
        }
    }
    int i[RUNS], j[RUNS];
#pragma unroll
    for (int r = 0; r < RUNS; ++r) { i[r] = lo[r]; j[r] = d0[r] - lo[r]; }
    for (int u = 0; u < E; ++u) {
        u64 a[RUNS], b[RUNS];
#pragma unroll
        for (int r = 0; r < RUNS; ++r) { a[r] = (A[i[r]] | orA) - subA; b[r] = B[j[r]] | orB; }   // sentinels stand in for an exhausted list
#pragma unroll
        for (int r = 0; r < RUNS; ++r) {
            const bool live = d0[r] + u < d1[r];
            const bool take_a = a[r] < b[r];
            if (live) out[d0[r] + u] = take_a ? a[r] : b[r];
            i[r] += (live && take_a) ? 1 : 0;
            j[r] += (live && !take_a) ? 1 : 0;
        }
    }
    if (lane == 0) out[n] = ~0ull;
}

// The same merge by a whole workgroup of `nthreads` threads (thread `tid` takes one run of consecutive
// outputs): for patches so long that a buffer pair per wavefront does not fit in LDS.  The caller puts
// a workgroup barrier behind it before anyone reads `out`.
__device__ __forceinline__ void block_merge(const u64* A, int nA, const u64* B, int nB, u64 orB, u64* out, int tid,
                                            int nthreads, u64 orA = 0, u64 subA = 0) {
    const int n = nA + nB;
    const int E = (n + nthreads - 1) / nthreads;
    const int d0 = min(tid * E, n), d1 = min(d0 + E, n);
    int lo = max(0, d0 - nB), hi = min(d0, nA);
    while (lo < hi) {                                          // co-rank of the run's first output
        const int mid = (lo + hi) >> 1;
        const bool a_first = ((A[mid] | orA) - subA) < (B[d0 - mid - 1] | orB);
        lo = a_first ? mid + 1 : lo;
        hi = a_first ? hi : mid;
    }
    int i = lo, j = d0 - lo;
    for (int e = d0; e < d1; ++e) {
        const u64 a = (A[i] | orA) - subA, b = B[j] | orB;     // sentinels stand in for an exhausted list
        const bool take_a = a < b;
        out[e] = take_a ? a : b;
        i += take_a ? 1 : 0;
        j += take_a ? 0 : 1;
    }
    if (tid == 0) out[n] = ~0ull;
}

constexpr int MERGE_THREADS = 256;
constexpr int MERGE_RUNS = 1;                             // runs of outputs a lane merges side by side
constexpr int MERGE_WAVES = MERGE_THREADS / kWave;

// One workgroup = TW consecutive patches of one output row.
//   pix_z / pix_c : every pixel's channels sorted ascending and their channel ids, rows of Cs entries
//   sorted / perm : [S, stride] outputs (entries past P padded with +inf / 0), n_real[S]
// BLOCKWIDE = false: every wavefront merges patches of its own between two buffers private to it.
// BLOCKWIDE = true (patches of thousands of entries, whose buffer pairs would not fit once per
// wavefront): the workgroup merges one patch at a time between a single pair of buffers.
template <int THREADS, bool BLOCKWIDE>
__global__ void __launch_bounds__(THREADS)
merge_patches_kernel(const float* __restrict__ pix_z, const int32_t* __restrict__ pix_c, int Cs,
                     float* __restrict__ sorted, int32_t* __restrict__ perm, int32_t* __restrict__ n_real,
                     int H, int W, int C, int Kh, int Kw, int Sh, int Sw, int Nh, int Nw, int TW, int tiles_w,
                     int stride, float max_cmp, int c4_shift, unsigned tile_cols_magic) {
    extern __shared__ __align__(16) unsigned char lds_raw[];
    const int tile_cols = (TW - 1) * Sw + Kw;
    const int KhC = Kh * C;
    const int P = KhC * Kw;
    // LDS carve-up (8-byte pieces first)
    // The pixel lists are dead once the column lists exist; the per-wave output staging reuses
    // their space.
    // lists end with a sentinel; a wavefront owns a buffer for the finished patch and one for the
    // list before it (the merges of a patch alternate between the two)
    const int col_stride = KhC + 1, out_stride = P + 1 + (Kw > 2 ? P - KhC + 1 : 0);
    u64* col_keys = reinterpret_cast<u64*>(lds_raw);                                   // [tile_cols][KhC + 1]
    u64* out_keys = col_keys + (size_t)tile_cols * col_stride;                         // [buffer pairs][out_stride]
    float* px_z = reinterpret_cast<float*>(out_keys);                                  // [Kh][tile_cols][C]
    uint16_t* px_c = reinterpret_cast<uint16_t*>(px_z + (size_t)Kh * tile_cols * C);   // [Kh][tile_cols][C]

    const int tile = blockIdx.x % tiles_w;
    const int rowid = blockIdx.x / tiles_w;
    const int nh = rowid % Nh, a = rowid / Nh;
    const int nw0 = tile * TW;
    const int w_first = nw0 * Sw;

    // Both passes below walk the pixel lists in groups of four channels: group g is channels
    // 4*(g % C4) .. +3 of pixel row g / C4 (row = kh * tile_cols + col).  The divisions by runtime
    // values are a shift (C4 a power of two, the usual case) and a multiply-high.
    const int C4 = C / 4;
    const int n_groups = Kh * tile_cols * C4;
    auto split = [&](int g, int& row, int& c, int& kh, int& col) {
        row = c4_shift >= 0 ? g >> c4_shift : g / C4;
        c = (g - row * C4) * 4;
        kh = (int)__umulhi((unsigned)row, tile_cols_magic);
        col = row - kh * tile_cols;
    };

    // ---- stage the sorted pixels under the tile ------------------------------------------------
    // loads are issued in batches: one at a time would cost a memory latency per group
    constexpr int STAGE = 4;
    for (int base = threadIdx.x; base < n_groups; base += STAGE * THREADS) {
        float4 zv[STAGE];
        int4 cv[STAGE];
#pragma unroll
        for (int u = 0; u < STAGE; ++u) {
            const int g = base + u * THREADS;
            int row, c, kh, col;
            split(g, row, c, kh, col);
            const int wp = w_first + col;
            zv[u] = make_float4(INFINITY, INFINITY, INFINITY, INFINITY);
            cv[u] = make_int4(c, c + 1, c + 2, c + 3);
            if (g < n_groups && wp < W) {
                const size_t src = ((size_t)(a * H + nh * Sh + kh) * W + wp) * Cs + c;
                zv[u] = *reinterpret_cast<const float4*>(pix_z + src);
                cv[u] = *reinterpret_cast<const int4*>(pix_c + src);
            }
        }
#pragma unroll
        for (int u = 0; u < STAGE; ++u) {
            const int g = base + u * THREADS;
            if (g < n_groups) {
                reinterpret_cast<float4*>(px_z)[g] = zv[u];
                reinterpret_cast<uint2*>(px_c)[g] = make_uint2((uint32_t)cv[u].x | ((uint32_t)cv[u].y << 16),
                                                               (uint32_t)cv[u].z | ((uint32_t)cv[u].w << 16));
            }
        }
    }
    __syncthreads();

    // ---- column lists: merge the Kh pixels of every column -----------------------------------------
    // A thread ranks the NB = 4 elements of a group side by side.
    for (int g = threadIdx.x; g < n_groups; g += THREADS) {
        int row, l0, kh, col;
        split(g, row, l0, kh, col);
        const float4 zq = reinterpret_cast<const float4*>(px_z)[g];
        const uint2 cq = reinterpret_cast<const uint2*>(px_c)[g];
        const float z[NB] = {zq.x, zq.y, zq.z, zq.w};
        const uint32_t ch[NB] = {cq.x & 0xffffu, cq.x >> 16, cq.y & 0xffffu, cq.y >> 16};
        int rank[NB];
#pragma unroll
        for (int i = 0; i < NB; ++i) rank[i] = l0 + i;
        for (int k2 = 0; k2 < kh; ++k2)          // pixels above: equal values come first there
            count_before_f32<false>(px_z + (size_t)(k2 * tile_cols + col) * C, C, z, rank);
        for (int k2 = kh + 1; k2 < Kh; ++k2)     // pixels below: only strictly smaller values precede
            count_before_f32<true>(px_z + (size_t)(k2 * tile_cols + col) * C, C, z, rank);
#pragma unroll
        for (int i = 0; i < NB; ++i)
            col_keys[(size_t)col * col_stride + rank[i]] = ((u64)order_key(z[i]) << 32) | ((u64)kh << 24) | ch[i];
    }
    __syncthreads();                                          // the pixel lists are dead from here on
    for (int col = threadIdx.x; col < tile_cols; col += THREADS) col_keys[(size_t)col * col_stride + KhC] = ~0ull;
    __syncthreads();

    if constexpr (BLOCKWIDE) {
        // ---- patches, one at a time, by the whole workgroup ------------------------------------------
        __shared__ int below_count;
        u64* other = out_keys + P + 1;
        const u64* acc = nullptr;
        auto store_patch = [&](int j) {                       // (entered and left by the whole workgroup)
            const size_t s = (size_t)(a * Nh + nh) * Nw + nw0 + j;
            float* so = sorted + s * stride;
            int32_t* po = perm + s * stride;
            int below = 0;
            for (int e = threadIdx.x; e < stride; e += THREADS) {
                float z = INFINITY;
                int32_t id = 0;
                if (e < P) {
                    const u64 key = acc[e];
                    z = order_key_to_float((uint32_t)(key >> 32));
                    const uint32_t low = (uint32_t)key;                    // kh | kw | c
                    id = (int32_t)(((low >> 24) * Kw + ((low >> 16) & 0xffu)) * C + (low & 0xffffu));
                }
                below += (e < P && z <= max_cmp) ? 1 : 0;
                so[e] = z;
                po[e] = id;
            }
#pragma unroll
            for (int d = kWave / 2; d > 0; d >>= 1) below += __shfl_xor(below, d, kWave);
            if (threadIdx.x % kWave == 0 && below != 0) atomicAdd(&below_count, below);
            __syncthreads();                                  // the buffers are free again, the count is complete
            if (threadIdx.x == 0) { n_real[s] = below_count; below_count = 0; }
            __syncthreads();
        };
        if (threadIdx.x == 0) below_count = 0;
        __syncthreads();
        const int n_patches = min(TW, Nw - nw0);
        if (Kw == 3 && Sw == 1) {
            // pairs of neighbouring patches share the merge of their two common columns (see the wavefront form below)
            constexpr u64 ONE_COLUMN = 1ull << 16;
            for (int j = 0; j < n_patches; j += 2) {
                const u64* cols = col_keys + (size_t)j * col_stride;
                if (j + 1 < n_patches) {
                    block_merge(cols + col_stride, KhC, cols + 2 * col_stride, KhC, 2 * ONE_COLUMN, other, threadIdx.x,
                                THREADS, ONE_COLUMN, 0);
                    __syncthreads();
                    block_merge(cols, KhC, other, 2 * KhC, 0, out_keys, threadIdx.x, THREADS);
                    __syncthreads();
                    acc = out_keys;
                    store_patch(j);
                    block_merge(other, 2 * KhC, cols + 3 * col_stride, KhC, 2 * ONE_COLUMN, out_keys, threadIdx.x, THREADS,
                                0, ONE_COLUMN);
                    __syncthreads();
                    store_patch(j + 1);
                } else {
                    block_merge(cols, KhC, cols + col_stride, KhC, ONE_COLUMN, other, threadIdx.x, THREADS);
                    __syncthreads();
                    block_merge(other, 2 * KhC, cols + 2 * col_stride, KhC, 2 * ONE_COLUMN, out_keys, threadIdx.x, THREADS);
                    __syncthreads();
                    acc = out_keys;
                    store_patch(j);
                }
            }
            return;
        }
        for (int j = 0; j < n_patches; ++j) {
            const u64* cols = col_keys + (size_t)(j * Sw) * col_stride;
            acc = cols;
            for (int kw = 1; kw < Kw; ++kw) {
                u64* dst = ((Kw - 1 - kw) & 1) ? other : out_keys;
                block_merge(acc, kw * KhC, cols + (size_t)kw * col_stride, KhC, (u64)kw << 16, dst, threadIdx.x, THREADS);
                __syncthreads();
                acc = dst;
            }
            store_patch(j);
        }
        return;
    }

    // ---- patches: merge the Kw columns of every patch ----------------------------------------------
    // From here on a wavefront works alone: the column lists are read-only and its two buffers are
    // its own, so no workgroup barrier is needed between its merges and its output.
    const int lane = threadIdx.x % kWave;
    const int wave = threadIdx.x / kWave;
    u64* my_out = out_keys + (size_t)wave * out_stride;
    auto store_patch = [&](int j) {
        const size_t s = (size_t)(a * Nh + nh) * Nw + nw0 + j;
        float* so = sorted + s * stride;
        int32_t* po = perm + s * stride;
        int below = 0;                                        // wave-uniform count of entries <= max_cmp
        for (int e = lane; e < stride; e += kWave) {
            float z = INFINITY;
            int32_t id = 0;
            if (e < P) {
                const u64 key = my_out[e];
                z = order_key_to_float((uint32_t)(key >> 32));
                const uint32_t low = (uint32_t)key;                    // kh | kw | c
                id = (int32_t)(((low >> 24) * Kw + ((low >> 16) & 0xffu)) * C + (low & 0xffffu));
            }
            below += __builtin_popcountll(__builtin_amdgcn_ballot_w64(e < P && z <= max_cmp));
            so[e] = z;
            po[e] = id;
        }
        if (lane == 0) n_real[s] = below;
    };
    u64* other = my_out + P + 1;
    const int n_patches = min(TW, Nw - nw0);
    if (Kw == 3 && Sw == 1) {
        // Neighbouring patches j and j + 1 share the columns j + 1 and j + 2: their merge M is made once,
        // with the column numbers of patch j in the keys (1 and 2), and serves both -- patch j is column j
        // merged with M, patch j + 1 is M, its column numbers lowered by one, merged with column j + 3.
        // Eight column lengths of sequential merging per pair of patches instead of ten.  (Keys are
        // distinct and the result of a merge is their ascending order, whatever was merged first.)
        // A wavefront takes a run of neighbouring patches, as long as the others' give or take one, in
        // pairs plus a single one where their number is odd.
        constexpr u64 ONE_COLUMN = 1ull << 16;
        constexpr int WAVES = THREADS / kWave;
        const int base = n_patches / WAVES, extra = n_patches - base * WAVES;
        const int j_first = wave * base + min(wave, extra), j_end = j_first + base + (wave < extra ? 1 : 0);
        for (int j = j_first; j < j_end; j += 2) {
            const u64* cols = col_keys + (size_t)j * col_stride;
            if (j + 1 < j_end) {
                wave_merge<MERGE_RUNS>(cols + col_stride, KhC, cols + 2 * col_stride, KhC, 2 * ONE_COLUMN, other, lane,
                                       ONE_COLUMN, 0);
                wave_merge<MERGE_RUNS>(cols, KhC, other, 2 * KhC, 0, my_out, lane);
                store_patch(j);
                wave_merge<MERGE_RUNS>(other, 2 * KhC, cols + 3 * col_stride, KhC, 2 * ONE_COLUMN, my_out, lane, 0,
                                       ONE_COLUMN);
                store_patch(j + 1);
            } else {
                wave_merge<MERGE_RUNS>(cols, KhC, cols + col_stride, KhC, ONE_COLUMN, other, lane);
                wave_merge<MERGE_RUNS>(other, 2 * KhC, cols + 2 * col_stride, KhC, 2 * ONE_COLUMN, my_out, lane);
                store_patch(j);
            }
        }
        return;
    }
    for (int j = wave; j < n_patches; j += THREADS / kWave) {
        // column 0 with 1, the result with 2, ...: the merge that takes in column kw writes the
        // patch buffer when Kw - 1 - kw is even and the other buffer otherwise, so that the last
        // one lands in the patch buffer
        const u64* cols = col_keys + (size_t)(j * Sw) * col_stride;
        const u64* acc = cols;
        for (int kw = 1; kw < Kw; ++kw) {
            u64* dst = ((Kw - 1 - kw) & 1) ? other : my_out;
            wave_merge<MERGE_RUNS>(acc, kw * KhC, cols + (size_t)kw * col_stride, KhC, (u64)kw << 16, dst, lane);
            acc = dst;
        }
        store_patch(j);
    }
}

// LDS of a workgroup with `pairs` buffer pairs for finished / half-finished patches.
size_t merge_lds_bytes(int C, int Kh, int Kw, int Sw, int TW, int pairs = MERGE_WAVES) {
    const size_t tile_cols = (size_t)(TW - 1) * Sw + Kw;
    const size_t KhC = (size_t)Kh * C, P = KhC * Kw;
    const size_t staging = (size_t)pairs * (P + 1 + (Kw > 2 ? P - KhC + 1 : 0)) * 8;
    const size_t pixels = (size_t)Kh * tile_cols * C * (4 + 2);
    return tile_cols * (KhC + 1) * 8 + (staging > pixels ? staging : pixels);
}

constexpr size_t MERGE_LDS_CAP = 160 * 1024;
constexpr int MERGE_BLOCKWIDE_THREADS = 1024;

// How a layer's patches are merged.  Patches per tile: as many as fit in 52 KB of LDS (so three
// workgroups share a CU), at most 16, never more than the row holds.  Layers with so many channels
// that not even two patches fit in 52 KB take what fits in MERGE_LDS_CAP (one workgroup per CU); where
// that leaves a narrow tile or none at all (a buffer pair per wavefront is 31 KB for 3 x 3 x 256 and
// 61 KB for 3 x 3 x 512), the workgroup -- of 16 wavefronts then -- keeps a single pair and merges one
// patch at a time, the row cut into tiles of equal width.
struct MergePlan {
    bool ok, blockwide;
    int tw;
    size_t lds;
    int waves = MERGE_WAVES;                               // wavefronts of a workgroup (each with a buffer pair)
};
MergePlan merge_plan(const ConvGeom& g) {
    const int C = (int)g.C, Kh = (int)g.Kh, Kw = (int)g.Kw, Sw = (int)g.Sw;
    const int tw_max = g.Nw < 16 ? (int)g.Nw : 16;
    int tw = tw_max;
    while (tw > 1 && merge_lds_bytes(C, Kh, Kw, Sw, tw) > 52 * 1024) --tw;
    if (tw < 2) {
        // one workgroup per CU: worth it while the tile stays wide (3 x 3 x 128: 16 patches; with 256
        // channels only 4 would fit, and the block-wide form below is faster: 145 against 186 us at 14 x 14)
        // (with eight wavefronts if their buffer pairs leave room for tiles of eight patches: 3 x 3 x 128 at
        // 28 x 28, 32 images: 237 against 318 us with four)
        int tw8 = tw_max;
        while (tw8 > 1 && merge_lds_bytes(C, Kh, Kw, Sw, tw8, 8) > MERGE_LDS_CAP) --tw8;
        if (tw8 >= 2 && tw8 >= (tw_max < 8 ? tw_max : 8) && merge_lds_bytes(C, Kh, Kw, Sw, tw8, 8) <= MERGE_LDS_CAP) {
            const int tiles = ((int)g.Nw + tw8 - 1) / tw8;
            tw8 = ((int)g.Nw + tiles - 1) / tiles;
            MergePlan p8{true, false, tw8, merge_lds_bytes(C, Kh, Kw, Sw, tw8, 8)};
            p8.waves = 8;
            return p8;
        }
        tw = tw_max;
        while (tw > 1 && merge_lds_bytes(C, Kh, Kw, Sw, tw) > MERGE_LDS_CAP) --tw;
        if (tw < (tw_max < 8 ? tw_max : 8)) tw = 1;
    }
    if (tw >= 2 && merge_lds_bytes(C, Kh, Kw, Sw, tw) <= MERGE_LDS_CAP)
        return MergePlan{true, false, tw, merge_lds_bytes(C, Kh, Kw, Sw, tw)};
    // (the block-wide form keeps a counter in static LDS next to the dynamic area)
    constexpr size_t CAP1 = MERGE_LDS_CAP - 64;
    tw = tw_max;
    while (tw > 1 && merge_lds_bytes(C, Kh, Kw, Sw, tw, 1) > CAP1) --tw;
    if (tw >= 2) {
        const int tiles = ((int)g.Nw + tw - 1) / tw;
        tw = ((int)g.Nw + tiles - 1) / tiles;
    }
    const size_t lds = merge_lds_bytes(C, Kh, Kw, Sw, tw, 1);
    return MergePlan{tw >= 2 && lds <= CAP1, true, tw, lds};
}

}  // namespace

// The merge path needs channel ids and kh in 16 bits, a useful amount of sharing and an LDS
// footprint within reach; everything else goes through the bitonic network.
bool merge_sort_supported(const ConvGeom& g) {
    if (g.C < 32 || g.C % NB != 0 || g.C > 4096 || g.Kw < 2 || g.Kh > 255 || g.Kw > 255) return false;
    return merge_plan(g).ok;
}

// One-time set-up on device `dev` (the current device): the dynamic-LDS limit of every
// instantiation, so that no later launch calls hipFuncSetAttribute (not allowed during capture).
int merge_prepare_device(int dev) {
    static std::atomic<bool> done[kMaxDevices];
    if (dev < 0 || dev >= kMaxDevices) return fail(SNNTC_ERR_UNSUPPORTED, "patch merge: device index %d not supported", dev);
    if (done[dev].load(std::memory_order_acquire)) return SNNTC_OK;
    SNNTC_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void*>(merge_patches_kernel<MERGE_THREADS, false>),
                                        hipFuncAttributeMaxDynamicSharedMemorySize, (int)MERGE_LDS_CAP));
    SNNTC_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void*>(merge_patches_kernel<2 * MERGE_THREADS, false>),
                                        hipFuncAttributeMaxDynamicSharedMemorySize, (int)MERGE_LDS_CAP));
    SNNTC_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void*>(merge_patches_kernel<MERGE_BLOCKWIDE_THREADS, true>),
                                        hipFuncAttributeMaxDynamicSharedMemorySize, (int)MERGE_LDS_CAP - 64));
    done[dev].store(true, std::memory_order_release);
    return SNNTC_OK;
}

int launch_merge_patches(const float* pix_z, const int32_t* pix_c, int64_t Cs, float* sorted, int32_t* perm,
                         int32_t* n_real, const ConvGeom& g, int64_t stride, float max_cmp,
                         hipStream_t stream) {
    const MergePlan plan = merge_plan(g);
    const int tw = plan.tw;
    const size_t lds = plan.lds;
    const int tiles_w = (int)((g.Nw + tw - 1) / tw);
    const int64_t blocks = g.B * g.Nh * tiles_w;
    if (blocks > 0x7fffffffLL) return fail(SNNTC_ERR_TOO_LARGE, "patch merge: grid too large");
    // C / 4 as a shift where it is a power of two; row / tile_cols as a multiply-high (exact for rows < 2^16)
    const int c4 = (int)g.C / 4;
    int c4_shift = -1;
    if ((c4 & (c4 - 1)) == 0) { c4_shift = 0; while ((1 << c4_shift) < c4) ++c4_shift; }
    const unsigned tile_cols = (unsigned)((tw - 1) * g.Sw + g.Kw);
    const unsigned magic = (unsigned)((0x100000000ull + tile_cols - 1) / tile_cols);
    int dev = 0;
    SNNTC_HIP_CHECK(hipGetDevice(&dev));
    const int prep = merge_prepare_device(dev);
    if (prep) return prep;
    {
        KernelTimerScope timer_("merge_patches", stream);
        if (plan.blockwide)
            hipLaunchKernelGGL((merge_patches_kernel<MERGE_BLOCKWIDE_THREADS, true>), dim3((unsigned)blocks),
                               dim3(MERGE_BLOCKWIDE_THREADS), lds, stream, pix_z, pix_c, (int)Cs, sorted, perm, n_real,
                               (int)g.H, (int)g.W, (int)g.C, (int)g.Kh, (int)g.Kw, (int)g.Sh, (int)g.Sw, (int)g.Nh,
                               (int)g.Nw, tw, tiles_w, (int)stride, max_cmp, c4_shift, magic);
        else if (plan.waves == 2 * MERGE_WAVES)
            hipLaunchKernelGGL((merge_patches_kernel<2 * MERGE_THREADS, false>), dim3((unsigned)blocks),
                               dim3(2 * MERGE_THREADS), lds, stream, pix_z, pix_c, (int)Cs, sorted, perm, n_real, (int)g.H,
                               (int)g.W, (int)g.C, (int)g.Kh, (int)g.Kw, (int)g.Sh, (int)g.Sw, (int)g.Nh, (int)g.Nw, tw,
                               tiles_w, (int)stride, max_cmp, c4_shift, magic);
        else
            hipLaunchKernelGGL((merge_patches_kernel<MERGE_THREADS, false>), dim3((unsigned)blocks), dim3(MERGE_THREADS),
                               lds, stream, pix_z, pix_c, (int)Cs, sorted, perm, n_real, (int)g.H, (int)g.W, (int)g.C,
                               (int)g.Kh, (int)g.Kw, (int)g.Sh, (int)g.Sw, (int)g.Nh, (int)g.Nw, tw, tiles_w,
                               (int)stride, max_cmp, c4_shift, magic);
    }
    SNNTC_HIP_CHECK(hipGetLastError());
    return SNNTC_OK;
}

}  // namespace snntc
