// Backward kernels specialised for conv layers: lanes are input channels (dX) or output channels (dW).
//
// Same contract as grad.hip (snntc/snncvgrad_kernels.cu.cc:15-161): with upm = grad*1/S, zero where
// y > MAX-0.1, and ym the spike times y themselves, patch s = (a, nh, nw), element i = (kh*Kw + kw)*C + c,
//   dXpad[a,h,w,c] = sum over patches covering (h,w) and over kc of [x <= ym[s,kc]] upm[s,kc] W[i,kc]
//   dW[i,kc]       = sum over patches of min(x_si - ym[s,kc], 0) * upm[s,kc]
// Both kernels put the channel (dX) or the output channel (dW) on the lanes, so everything that
// depends only on the patch is wave-uniform and is fetched through the scalar path.
#include "snntc_common.h"
#include <type_traits>

namespace snntc {
namespace {

// ---------------------------------------------------------------------------------------------
// dX.  A wavefront owns TILE consecutive pixels of one image row and 64 channels (fewer channels: more
// tiles, see MULTI); lane = channel.  Tap-major sweep (any kernel width): for every kernel tap (kh, kw) the
// lane keeps its weight row W[(kh,kw,c), 0..KCB) in registers and sweeps the tile; the patch under the tap is
// the same for all lanes.  Slot-major sweep (three-column kernels): see KW below.  The weights come
// from a copy of W regrouped as [tap][kc / 4][c][kc % 4] (written by backward_prologue_kernel): read from W itself,
// every 16-byte fetch of a wavefront touches 64 different cache lines instead of 8.  The ym / upm
// rows of the TILE + Kw - 1 patches one kernel row can touch are staged in a wavefront-private
// piece of LDS (lane = output channel while staging) and read back as broadcasts, four output
// channels per read.  Gather form: no atomics, fixed summation order.
//
// The mask x <= ym is evaluated arithmetically (dx_mac8).  That is exact while MAX_SPIKE_TIME is at
// most 2^86 and no two unequal spike times lie closer together than 1 / dx_mask_scale (2^-109 for
// MAX_SPIKE_TIME = 1e5): differences that small exist only between values below 2^-85.
// ---------------------------------------------------------------------------------------------
constexpr int DX_TILE = 8;
constexpr int DX_WAVES3 = 4;           // wavefronts per SIMD the KW = 3 variant is compiled for

// Eight masked MACs  acc += upm_k * (x <= ym_k ? w_k : 0)  without a compare or a select: with
//   m = clamp01(x * BIG - ym_k * BIG)       (one fused multiply-add with the clamp output modifier)
// m is exactly 1 where x > ym_k and exactly 0 where x <= ym_k: the fused operation rounds the exact
// value of (x - ym_k) * BIG, whose sign is that of x - ym_k, and BIG (dx_mask_scale) is large enough
// that the smallest difference two unequal spike times can have maps to at least 1 while MAX * BIG stays finite.
// Then t = w_k - m * w_k is w_k or 0 (both exact) and acc += upm_k * t.  All three are plain
// multiply-adds on vector registers, which this chip issues faster than compares, selects and DPP
// operands (about 2.8 against 4.2 cycles each with several wavefronts per SIMD).  ny_k = -ym_k * BIG
// (+inf for outputs that take no part, so m = 1) and upm_k arrive as broadcast LDS reads.  The
// schedule keeps every result two other instructions away from its first use.
#define SNNTC_DX_M(K, T) "v_fma_f32 %[" #T "], %[x], %[big], %[y" #K "] clamp\n"
#define SNNTC_DX_T(K, T) "v_fma_f32 %[" #T "], -%[" #T "], %[w" #K "], %[w" #K "]\n"
#define SNNTC_DX_F(K, T) "v_fmac_f32_e32 %[acc], %[u" #K "], %[" #T "]\n"

__device__ __forceinline__ void dx_mac8(float& acc, float x, float big, const float* u, const float* y,
                                        const float* w) {
    float ta, tb, tc;
    asm volatile(
        SNNTC_DX_M(0, ta)
        SNNTC_DX_M(1, tb) SNNTC_DX_T(0, ta)
        SNNTC_DX_M(2, tc) SNNTC_DX_T(1, tb) SNNTC_DX_F(0, ta)
        SNNTC_DX_M(3, ta) SNNTC_DX_T(2, tc) SNNTC_DX_F(1, tb)
        SNNTC_DX_M(4, tb) SNNTC_DX_T(3, ta) SNNTC_DX_F(2, tc)
        SNNTC_DX_M(5, tc) SNNTC_DX_T(4, tb) SNNTC_DX_F(3, ta)
        SNNTC_DX_M(6, ta) SNNTC_DX_T(5, tc) SNNTC_DX_F(4, tb)
        SNNTC_DX_M(7, tb) SNNTC_DX_T(6, ta) SNNTC_DX_F(5, tc)
        SNNTC_DX_T(7, tb) SNNTC_DX_F(6, ta)
        SNNTC_DX_F(7, tb)
        : [acc] "+v"(acc), [ta] "=&v"(ta), [tb] "=&v"(tb), [tc] "=&v"(tc)
        : [x] "v"(x), [big] "v"(big), [y0] "v"(y[0]), [y1] "v"(y[1]), [y2] "v"(y[2]), [y3] "v"(y[3]), [y4] "v"(y[4]),
          [y5] "v"(y[5]), [y6] "v"(y[6]), [y7] "v"(y[7]), [u0] "v"(u[0]), [u1] "v"(u[1]), [u2] "v"(u[2]),
          [u3] "v"(u[3]), [u4] "v"(u[4]), [u5] "v"(u[5]), [u6] "v"(u[6]), [u7] "v"(u[7]), [w0] "v"(w[0]),
          [w1] "v"(w[1]), [w2] "v"(w[2]), [w3] "v"(w[3]), [w4] "v"(w[4]), [w5] "v"(w[5]), [w6] "v"(w[6]),
          [w7] "v"(w[7]));
}

// MULTI is for layers with at most 32 input channels: the wavefront is cut into 2, 4, 8 or 16 parts
// of 32, 16, 8 or 4 lanes (`1 << parts_shift` of them) that take the same channels of as many neighbouring
// 8-pixel tiles, so few lanes idle.  Which patch lies under a tap then differs between the parts; a
// part whose patch does not exist reads a slot that holds (ym, upm) = (-inf, 0) -- +inf in the scaled form
// of dx_mac8 -- and so adds nothing.
//
// KW = 3 (the layer's kernel is three columns wide; 0: any width): the sweep is turned inside out.  A slot's
// operands are read once per DX_GK output channels and serve the up to three (pixel, tap) pairs that meet
// that patch, with the weights of all three taps of those channels in registers.  That takes far fewer
// registers than a whole weight row per tap; they go into a second set of weights and of slot operands,
// fetched while the current ones are in use, and fewer LDS reads are needed (80 instead of 192 per tile and
// 16 output channels).
constexpr int DX_GK = 8;
template <int KCB, bool MULTI, int KW>
__global__ void __launch_bounds__(256)
    __attribute__((amdgpu_waves_per_eu(KW == 3 ? DX_WAVES3 : KCB == 64 && MULTI ? 3 : 4)))
cv_grad_input_chan_kernel(const float* __restrict__ xpad, const float* __restrict__ wq,
                          const float* __restrict__ upm, const float* __restrict__ ym,
                          float* __restrict__ dx, CropGeom crop, int H, int W, int C, int Kc, int Kh, int Kw, int Sh,
                          int Sw, int Nh, int Nw, int tiles_w, int c_blocks, int64_t n_items, int64_t lead_items,
                          int lead_blocks, float max_cmp, int ksplit, float big, int parts_shift) {
    extern __shared__ __align__(16) float staged[];      // per wavefront: [2][n_slots + 1][KCB]; ksplit > 1: then `partial`
    const int parts = MULTI ? 1 << parts_shift : 1;
    const int span = DX_TILE * parts;                    // pixels of one wavefront
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
    // ksplit = 1: a tile per single-wavefront workgroup.  ksplit = 2 or 4 (layers with few tiles and many
    // output channels): a tile per workgroup of that many wavefronts, each takes its share of the output
    // channels and their sums are added in wavefront order.
    // Items are (image, row, tile, channel block).  When the last tile of a row is a partial one, those
    // tiles form a second run of workgroups behind all others (`lead_blocks` workgroups, a multiple of
    // the XCD count, hold the `lead_items` others), so that the launch ends on its shortest items and
    // the CUs drain together.  Both runs are numbered XCD-contiguously: an XCD works on the same
    // rows in both, and on neighbouring tiles, which share their staged rows, one after another.
    const bool lead = (int)blockIdx.x < lead_blocks;
    const int64_t item = lead ? xcd_contiguous(blockIdx.x, lead_blocks)
                              : xcd_contiguous(blockIdx.x - lead_blocks, gridDim.x - lead_blocks);
    const int ks = wave;                                 // 0 without the split
    if (item >= (lead ? lead_items : n_items - lead_items)) return;
    const int lane = threadIdx.x % kWave;
    const int part = MULTI ? lane >> (6 - parts_shift) : 0;
    const int tiles_lead = lead_items < n_items ? tiles_w - 1 : tiles_w;
    const int cb = (int)(item % c_blocks);
    int64_t rest = item / c_blocks;
    int tw = tiles_w - 1;
    if (lead) { tw = (int)(rest % tiles_lead); rest /= tiles_lead; }
    const int h = (int)(rest % H);
    const int a = (int)(rest / H);
    const int w0 = tw * span;                            // first pixel of the wavefront
    const int p0 = w0 + part * DX_TILE;                  // first pixel of this lane
    const int c = MULTI ? (lane & ((kWave >> parts_shift) - 1)) : cb * kWave + lane;
    const bool lane_ok = c < C;
    const unsigned cc = (unsigned)(lane_ok ? c : C - 1);
    const int n_slots = span + Kw - 1;                   // slot d: the patch whose left column is w0-Kw+1+d
    float* __restrict__ ys = staged + (size_t)wave * 2 * (n_slots + 1) * KCB;
    float* __restrict__ us = ys + (n_slots + 1) * KCB;
    if (lane < KCB) {                                    // the spare slot
        ys[n_slots * KCB + lane] = INFINITY;             // in the scaled form the loop below produces
        us[n_slots * KCB + lane] = 0.0f;
    }

    // Pixels that need no work: those outside the window of the gradient the caller wants (with the
    // window of the un-padded image that is the whole SAME border: 11 % of a 34 x 34 padded image, 40 %
    // of a 9 x 9 one) and padded pixels anywhere (x > MAX-0.1 can never satisfy x <= ym).  `live` has
    // bit t set when pixel t of some lane's tile has work; a wavefront whose row lies outside the
    // window has none at all (with ksplit > 1 that holds for the whole workgroup).
    const int oh = h - crop.top;
    if (oh < 0 || oh >= crop.h) return;
    float xv[DX_TILE], acc[DX_TILE];
    unsigned live = 0;
    const float* __restrict__ xrow = xpad + ((size_t)(a * H + h) * W) * C + cc;
#pragma unroll
    for (int t = 0; t < DX_TILE; ++t) {
        const int wx = min(p0 + t, W - 1);
        xv[t] = xrow[(size_t)wx * C];
        acc[t] = 0.0f;
        const int ow = p0 + t - crop.left;
        if (__any(xv[t] <= max_cmp && ow >= 0 && ow < crop.w)) live |= 1u << t;
    }
    // KW = 3: slots that hold no patch are filled with (+inf, 0), a term that adds nothing, so a lane may read
    // any slot.  With a column stride of 1 those are the slots outside [slot_lo, slot_hi): they are filled once and
    // left alone by the rescaling pass of every staging round; otherwise they are filled again after every round.
    // Bit 3 * d + kw of `work` says that the d-th slot of a part and tap kw meet a pixel with work (for some lane).
    auto slot_exists = [&](int sl) {
        const int ww = w0 - Kw + 1 + sl;
        if (ww < 0) return false;
        return Sw == 1 ? ww < Nw : (ww % Sw == 0 && ww / Sw < Nw);
    };
    auto fill_empty_slots = [&]() {
        for (int sl = 0; sl < n_slots; ++sl)
            if (!slot_exists(sl) && lane < KCB) { ys[sl * KCB + lane] = INFINITY; us[sl * KCB + lane] = 0.0f; }
    };
    const int slot_lo = max(0, Kw - 1 - w0), slot_hi = min(n_slots, Nw + Kw - 1 - w0);
    unsigned work = 0;
    float bigv = big;
    if constexpr (KW == 3) {
#pragma unroll
        for (int d = 0; d < DX_TILE + 2; ++d) {
            bool any_patch = false;
            for (int pt = 0; pt < parts; ++pt) any_patch = any_patch || slot_exists(d + pt * DX_TILE);
#pragma unroll
            for (int kw = 0; kw < 3; ++kw) {
                const int t = d - 2 + kw;                                 // the pixel that meets it under tap kw
                if (t >= 0 && t < DX_TILE && any_patch && (live >> t & 1u)) work |= 1u << (3 * d + kw);
            }
        }
        if (Sw == 1) fill_empty_slots();
    }
    asm volatile("v_mov_b32 %0, %1" : "=v"(bigv) : "s"(big));             // one register for all the blocks below
    if (live != 0) {
        for (int kh = 0; kh < Kh; ++kh) {
            const int hh = h - kh;
            if (hh < 0 || hh % Sh != 0) continue;
            const int nh = hh / Sh;
            if (nh >= Nh) continue;
            const size_t row0 = (size_t)(a * Nh + nh) * Nw;
            const int kc_share = Kc / ksplit;
            for (int kc0 = ks * kc_share; kc0 < (ks + 1) * kc_share; kc0 += KCB) {
                // stage the patch row (only slots whose patch exists are loaded)
                __builtin_amdgcn_wave_barrier();
                // The rows go from memory straight into LDS (buffer loads with the LDS bit: lane l of a load
                // writes dword l behind the load's LDS base).  A load covers 64 / KCB neighbouring slots --
                // with fewer than 64 output channels per slot the lanes share them out -- and all loads of
                // a round are in flight together.  No registers are involved, which the compiler used to
                // free by spilling the accumulators around this loop.
                constexpr int PER = kWave / KCB;
                const int sub = lane / KCB, kcl = lane - sub * KCB;
                const int row_bytes = (int)(((size_t)Nw * Kc - kc0) * sizeof(float));
                const __amdgpu_buffer_rsrc_t ybuf = __builtin_amdgcn_make_buffer_rsrc(
                    const_cast<float*>(ym + row0 * Kc + kc0), 0, row_bytes, 0x00020000);
                const __amdgpu_buffer_rsrc_t ubuf = __builtin_amdgcn_make_buffer_rsrc(
                    const_cast<float*>(upm + row0 * Kc + kc0), 0, row_bytes, 0x00020000);
                typedef __attribute__((address_space(3))) void lds_void;
                for (int d0 = 0; d0 < n_slots; d0 += PER) {
                    const int d = d0 + sub;
                    const int ww = w0 - Kw + 1 + d;
                    const int col = Sw == 1 ? ww : ww / Sw;
                    if (d < n_slots && ww >= 0 && (Sw == 1 || ww % Sw == 0) && col < Nw) {
                        const int so = (col * Kc + kcl) * (int)sizeof(float);
                        __builtin_amdgcn_raw_ptr_buffer_load_lds(ybuf, (lds_void*)(ys + d0 * KCB), 4, so, 0, 0, 0);
                        __builtin_amdgcn_raw_ptr_buffer_load_lds(ubuf, (lds_void*)(us + d0 * KCB), 4, so, 0, 0, 0);
                    }
                }
                asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
                __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
                __builtin_amdgcn_wave_barrier();
                // ym -> -ym * BIG, the operand of dx_mac8 (-inf, an output that takes no part, becomes +inf).
                // Slots that were not loaded: the tap-major sweep never reads them (it reads the spare slot
                // instead), the slot-major one reads them as (+inf, 0), see fill_empty_slots
                for (int i = lane; i < n_slots * (KCB / 4); i += kWave) {
                    if (KW == 3 && Sw == 1 && (i / (KCB / 4) < slot_lo || i / (KCB / 4) >= slot_hi)) continue;
                    float4 v4 = reinterpret_cast<float4*>(ys)[i];
                    v4.x *= -big; v4.y *= -big; v4.z *= -big; v4.w *= -big;
                    reinterpret_cast<float4*>(ys)[i] = v4;
                }
                if (KW == 3 && Sw != 1) fill_empty_slots();
                __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
                __builtin_amdgcn_wave_barrier();
                if constexpr (KW == 3) {
                    // wq[tap][kc / 4][c][kc % 4]: the 16-byte pieces the lanes fetch together are neighbours
                    // in memory.  Two register sets: the weights of the next DX_GK output channels are
                    // fetched while the current ones are in use.
                    const float4* __restrict__ wbase =
                        reinterpret_cast<const float4*>(wq) + ((size_t)(kh * 3) * (Kc / 4) + kc0 / 4) * C + cc;
                    const size_t tap_stride = (size_t)(Kc / 4) * C;
                    auto load_w = [&](float (&wr)[3][DX_GK], int g) {
#pragma unroll
                        for (int kw = 0; kw < 3; ++kw)
#pragma unroll
                            for (int q = 0; q < DX_GK; q += 4) {
                                const float4 v4 = wbase[kw * tap_stride + (size_t)(g * (DX_GK / 4) + q / 4) * C];
                                wr[kw][q] = v4.x; wr[kw][q + 1] = v4.y; wr[kw][q + 2] = v4.z; wr[kw][q + 3] = v4.w;
                            }
                    };
                    const float* __restrict__ ybase = ys + part * DX_TILE * KCB;
                    const int US = (span + 3) * KCB;                      // from a slot's ym row to its upm row
                    auto read_slot = [&](const float* __restrict__ yg, int d, float (&yd)[DX_GK], float (&ud)[DX_GK]) {
#pragma unroll
                        for (int v = 0; v < DX_GK; v += 4) {
                            const float4 y4 = *reinterpret_cast<const float4*>(yg + d * KCB + v);
                            const float4 u4 = *reinterpret_cast<const float4*>(yg + US + d * KCB + v);
                            yd[v] = y4.x; yd[v + 1] = y4.y; yd[v + 2] = y4.z; yd[v + 3] = y4.w;
                            ud[v] = u4.x; ud[v + 1] = u4.y; ud[v + 2] = u4.z; ud[v + 3] = u4.w;
                        }
                    };
                    // all slots of a half against the three taps of DX_GK output channels; the operands of the
                    // next slot are read while the current one computes
                    auto sweep = [&](const float (&wr)[3][DX_GK], const float* __restrict__ yg) {
                        float yq[2][DX_GK], uq[2][DX_GK];
                        // the bits are tested where they are used: as thirty loop-invariant conditions they would
                        // take sixty scalar registers
                        unsigned wk = work;
                        asm volatile("" : "+s"(wk));
                        read_slot(yg, 0, yq[0], uq[0]);
#pragma unroll
                        for (int d = 0; d < DX_TILE + 2; ++d) {
                            if (d + 1 < DX_TILE + 2) read_slot(yg, d + 1, yq[(d + 1) & 1], uq[(d + 1) & 1]);
                            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                            for (int kw = 0; kw < 3; ++kw) {
                                const int t = d - 2 + kw;
                                if (t < 0 || t >= DX_TILE) continue;
                                if (wk >> (3 * d + kw) & 1u) dx_mac8(acc[t], xv[t], bigv, uq[d & 1], yq[d & 1], wr[kw]);
                            }
                            __builtin_amdgcn_sched_barrier(0);
                        }
                    };
                    float wa[3][DX_GK], wb[3][DX_GK];
                    load_w(wa, 0);
#pragma unroll 1
                    for (int g = 0; g < KCB / DX_GK; g += 2) {
                        load_w(wb, g + 1);
                        sweep(wa, ybase + g * DX_GK);
                        if (g + 2 < KCB / DX_GK) load_w(wa, g + 2);
                        sweep(wb, ybase + (g + 1) * DX_GK);
                    }
                    continue;
                }
                for (int kw = 0; kw < Kw; ++kw) {
                    // wq[tap][kc / 4][c][kc % 4]: the 16-byte pieces the lanes fetch together are
                    // neighbours in memory
                    const float4* __restrict__ wrow =
                        reinterpret_cast<const float4*>(wq) + ((size_t)(kh * Kw + kw) * (Kc / 4) + kc0 / 4) * C + cc;
                    float wreg[KCB];
#pragma unroll
                    for (int q = 0; q < KCB; q += 4) {
                        const float4 v4 = wrow[(size_t)(q / 4) * C];
                        wreg[q] = v4.x; wreg[q + 1] = v4.y; wreg[q + 2] = v4.z; wreg[q + 3] = v4.w;
                    }
#pragma unroll
                    for (int t = 0; t < DX_TILE; ++t) {
                        const int ww = p0 + t - kw;
                        // (no division for the usual column stride of 1)
                        const bool has_patch = p0 + t < W && ww >= 0 && (Sw == 1 ? ww < Nw : (ww % Sw == 0 && ww / Sw < Nw));
                        if (!(live >> t & 1) || !__any(has_patch)) continue;
                        int slot = has_patch ? p0 + t - w0 - kw + Kw - 1 : n_slots;
                        if (!MULTI) slot = __builtin_amdgcn_readfirstlane(slot);   // same for every lane
                        const float* __restrict__ yrow = ys + slot * KCB;
                        const float* __restrict__ urow = us + slot * KCB;
                        // groups of 16 output channels: eight broadcast reads, then 48 multiply-adds
#pragma unroll
                        for (int g = 0; g < KCB / 16; ++g) {
                            float yq[16], uq[16];
#pragma unroll
                            for (int v = 0; v < 16; v += 4) {
                                const float4 y4 = *reinterpret_cast<const float4*>(yrow + g * 16 + v);
                                const float4 u4 = *reinterpret_cast<const float4*>(urow + g * 16 + v);
                                yq[v] = y4.x; yq[v + 1] = y4.y; yq[v + 2] = y4.z; yq[v + 3] = y4.w;
                                uq[v] = u4.x; uq[v + 1] = u4.y; uq[v + 2] = u4.z; uq[v + 3] = u4.w;
                            }
                            __builtin_amdgcn_sched_barrier(0);
                            dx_mac8(acc[t], xv[t], bigv, &uq[0], &yq[0], &wreg[g * 16]);
                            dx_mac8(acc[t], xv[t], bigv, &uq[8], &yq[8], &wreg[g * 16 + 8]);
                        }
                    }
                }
            }
        }
    }
    if (ksplit > 1) {                                     // block-uniform: all four wavefronts hold the same tile
        // sums of wavefronts 1..ksplit-1, [ksplit - 1][DX_TILE][64], behind the staging areas
        float* __restrict__ partial = staged + (size_t)(blockDim.x / kWave) * 2 * (n_slots + 1) * KCB;
        if (ks > 0) {
#pragma unroll
            for (int t = 0; t < DX_TILE; ++t) partial[((ks - 1) * DX_TILE + t) * kWave + lane] = acc[t];
        }
        __syncthreads();
        if (ks > 0) return;
        for (int v = 1; v < ksplit; ++v) {                // in wavefront order
#pragma unroll
            for (int t = 0; t < DX_TILE; ++t) acc[t] += partial[((v - 1) * DX_TILE + t) * kWave + lane];
        }
    }
    // only the pixels inside the caller's window of the padded image are stored
    if (lane_ok) {
        float* __restrict__ orow = dx + ((size_t)(a * crop.h + oh) * crop.w) * C + c;
#pragma unroll
        for (int t = 0; t < DX_TILE; ++t) {
            const int ow = p0 + t - crop.left;
            if (p0 + t < W && ow >= 0 && ow < crop.w) orow[(size_t)ow * C] = acc[t];
        }
    }
}

// ---------------------------------------------------------------------------------------------
// dW.  Lane = output channel kc.  The weight rows of one kernel row kh, (kw, c) flattened, are
// Kw*C consecutive floats of the padded image for every patch; a block owns up to DWW_RI
// consecutive ones, so the x values of a patch are one contiguous scalar fetch.  The patch range is cut into gridDim.z slices (partial sums are added in
// slice order afterwards) and each slice over the four wavefronts of the block.
// ---------------------------------------------------------------------------------------------
constexpr int DWW_RI = 32;

// FULL: every block has all DWW_RI rows (Kw*C is a multiple of it); the partial-block code is left out.
// R: rows a block works on (DWW_RI, or the multiple of 8 above Kw*C for layers whose kernel rows are
// shorter than that, e.g. 24 for a 7x7 stem on 3 channels: rows past the block's last one cost
// instructions like any other).
template <bool FULL, int R>
__global__ void __launch_bounds__(256)
cv_grad_weight_wide_kernel(const float* __restrict__ xpad, const float* __restrict__ upm,
                           const float* __restrict__ ym, float* __restrict__ dst, int S, int Kc, int rows,
                           int seg_per_slice, int H, int W, int C, int Kw, int Sh, int Sw, int Nh, int Nw,
                           int bias_row, float biasvolt, int s_safe, float neg_s, float post) {
    __shared__ float red[3][R + 1][kWave];
    const int lane = threadIdx.x % kWave;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
    const int j = blockIdx.x * kWave + lane;
    const unsigned jc = (unsigned)min(j, Kc - 1);
    const int KwC = Kw * C;
    const int chunks = (KwC + DWW_RI - 1) / DWW_RI;     // blocks per kernel row
    const int kh = blockIdx.y / chunks;
    const int q0 = (blockIdx.y - kh * chunks) * DWW_RI; // first (kw, c) of the block
    const int n_rows = min(DWW_RI, KwC - q0);
    const int i0 = kh * KwC + q0;                       // first weight row of the block

    const int s_begin = blockIdx.z * seg_per_slice;
    const int s_end = min(S, s_begin + seg_per_slice);
    const int per_wave = (s_end - s_begin + 3) / 4;
    const int s_lo = s_begin + wave * per_wave;
    const int s_hi = min(s_end, s_lo + per_wave);

    float acc[R];
#pragma unroll
    for (int r = 0; r < R; ++r) acc[r] = 0.0f;
    // the block of rows 0..31 also carries the bias row (x = biasvolt for every patch)
    const bool with_bias = bias_row >= 0 && blockIdx.y == 0;
    float acc_bias = 0.0f;

    if (s_lo < s_hi) {
        const int per_img = Nh * Nw;
        const int a = s_lo / per_img;
        const int r2 = s_lo - a * per_img;
        int nh = r2 / Nw, nw = r2 - nh * Nw;
        // the block's first input of patch s_lo; the step to the next patch is one add, plus one more
        // at the end of an output row and of an image
        const float* xb = xpad + ((size_t)(a * H + nh * Sh + kh) * W + (size_t)(nw * Sw)) * C + q0;
        const ptrdiff_t step_w = (ptrdiff_t)Sw * C;
        const ptrdiff_t wrap_w = ((ptrdiff_t)Sh * W - (ptrdiff_t)Nw * Sw) * C;
        const ptrdiff_t wrap_h = ((ptrdiff_t)H - (ptrdiff_t)Nh * Sh) * W * C;
        // y and up of the next patch are requested before the current one is worked on
        // (through buffer descriptors of the wavefront's patch range: a scalar running offset plus the
        // lane's constant column offset, no vector address arithmetic)
        const int range_bytes = (int)min((int64_t)(s_hi - s_lo) * Kc * (int64_t)sizeof(float), (int64_t)0x7ffffffc);
        const __amdgpu_buffer_rsrc_t ybuf =
            __builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(ym + (size_t)s_lo * Kc), 0, range_bytes, 0x00020000);
        const __amdgpu_buffer_rsrc_t ubuf =
            __builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(upm + (size_t)s_lo * Kc), 0, range_bytes, 0x00020000);
        const int col_bytes = (int)(jc * sizeof(float)), patch_bytes = Kc * (int)sizeof(float);
        int next_bytes = 0;
        float y_next = __uint_as_float(__builtin_amdgcn_raw_buffer_load_b32(ybuf, col_bytes, 0, 0));
        float u_next = __uint_as_float(__builtin_amdgcn_raw_buffer_load_b32(ubuf, col_bytes, 0, 0));
        // A block at the end of a kernel row fetches past its rows (the values are discarded), except
        // for the last few patches of the tensor, where that fetch could leave it: there the unused
        // rows re-read the block's last row.  Two loops, so that neither carries the other's code.
        const int s_fast = (FULL || n_rows == R) ? s_hi : max(s_lo, min(s_hi, s_safe));
        auto patches = [&](int s_from, int s_to, auto clamp_rows) {
            for (int s = s_from; s < s_to; ++s) {
                const float yv = y_next * -neg_s, uv = u_next;
                if (s + 1 < s_hi) next_bytes += patch_bytes;
                y_next = __uint_as_float(__builtin_amdgcn_raw_buffer_load_b32(ybuf, col_bytes, next_bytes, 0));
                u_next = __uint_as_float(__builtin_amdgcn_raw_buffer_load_b32(ubuf, col_bytes, next_bytes, 0));
#pragma unroll
                for (int r = 0; r < R; ++r) {
                    const float xv = decltype(clamp_rows)::value ? xb[min(r, n_rows - 1)] : xb[r];
                    acc[r] = __fmaf_rn(scaled_lead(xv, neg_s, yv), uv, acc[r]);
                }
                if (with_bias) {                          // block-uniform: a branch, not a select
                    asm volatile("");
                    acc_bias = __fmaf_rn(scaled_lead(biasvolt, neg_s, yv), uv, acc_bias);
                }
                xb += step_w;
                if (++nw == Nw) {
                    nw = 0; xb += wrap_w;
                    if (++nh == Nh) { nh = 0; xb += wrap_h; }
                }
            }
        };
        patches(s_lo, s_fast, std::false_type{});
        if (!FULL) patches(s_fast, s_hi, std::true_type{});
    }
    if (wave > 0) {
#pragma unroll
        for (int r = 0; r < R; ++r) red[wave - 1][r][lane] = acc[r];
        red[wave - 1][R][lane] = acc_bias;
    }
    __syncthreads();
    if (wave == 0 && j < Kc) {
        float* out = dst + (size_t)blockIdx.z * rows * Kc;
#pragma unroll
        for (int r = 0; r < R; ++r)
            if (r < n_rows)
                out[(size_t)(i0 + r) * Kc + j] =
                    (((acc[r] + red[0][r][lane]) + red[1][r][lane]) + red[2][r][lane]) * post;
        if (with_bias)
            out[(size_t)bias_row * Kc + j] =
                (((acc_bias + red[0][R][lane]) + red[1][R][lane]) + red[2][R][lane]) * post;
    }
}

// ---------------------------------------------------------------------------------------------
// dW for layers with at most 32 output channels.  Lane = (half, kc): the two halves of a wavefront
// take alternate patches, so no lane idles.  The 32 inputs of a patch that a block's rows need are
// fetched two per lane (lane r of the first 16 lanes of a half fetches inputs r and 16 + r of the half's own
// patch), left in a 256-byte buffer of the wavefront in LDS and read back by every lane of the half as
// eight 16-byte broadcasts: with the inputs in vector registers a term is the two plain multiply-adds of
// the wide kernel (scaled_lead), where a DPP operand, a minimum and a multiply-add used to cost twice
// the issue time.  Partial sums of the halves and of the four wavefronts are added in a fixed order
// through LDS.
// ---------------------------------------------------------------------------------------------
__global__ void __launch_bounds__(256)
cv_grad_weight_narrow_kernel(const float* __restrict__ xpad, const float* __restrict__ upm,
                             const float* __restrict__ ym, float* __restrict__ dst, int S, int Kc, int rows,
                             int seg_per_slice, int H, int W, int C, int Kw, int Sh, int Sw, int Nh, int Nw,
                             int bias_row, float biasvolt, int /*s_safe*/, float neg_s, float post) {
    __shared__ float red[4][DWW_RI + 1][kWave];
    __shared__ __align__(16) float xstage[4][2][DWW_RI];   // [wavefront][half][input]
    const int lane = threadIdx.x % kWave;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
    const int half = lane >> 5, kc = lane & 31;
    const unsigned jc = (unsigned)min(kc, Kc - 1);
    const int KwC = Kw * C;
    const int chunks = (KwC + DWW_RI - 1) / DWW_RI;
    const int kh = blockIdx.y / chunks;
    const int q0 = (blockIdx.y - kh * chunks) * DWW_RI;
    const int n_rows = min(DWW_RI, KwC - q0);
    const int i0 = kh * KwC + q0;

    const int s_begin = blockIdx.z * seg_per_slice;
    const int s_end = min(S, s_begin + seg_per_slice);
    const int per_wave = (s_end - s_begin + 3) / 4;
    const int s_lo = s_begin + wave * per_wave;
    const int s_hi = min(s_end, s_lo + per_wave);

    float acc[DWW_RI];
#pragma unroll
    for (int r = 0; r < DWW_RI; ++r) acc[r] = 0.0f;
    const bool with_bias = bias_row >= 0 && blockIdx.y == 0;
    float acc_bias = 0.0f;

    if (s_lo < s_hi) {
        const int per_img = Nh * Nw;
        // This lane's patch: s_lo + half, then every second one.  Its two inputs, ym and upm are followed
        // by pointers that move by adds alone (a step of two patches, plus the wraps at the end of an
        // output row and of an image), and the values of the next patch are requested before the
        // current one is worked on.  A lane past its last patch keeps pointing at it, with upm = 0.
        int s = s_lo + half;
        const int sc = min(s, s_hi - 1);
        const int a = sc / per_img;
        const int r2 = sc - a * per_img;
        int nh = r2 / Nw, nw = r2 - nh * Nw;
        const int l16 = lane & 15;                       // rows past the block's last one re-read it
        const float* px0 = xpad + ((size_t)(a * H + nh * Sh + kh) * W + (size_t)(nw * Sw)) * C + q0 + min(l16, n_rows - 1);
        const ptrdiff_t second = min(l16 + 16, n_rows - 1) - min(l16, n_rows - 1);
        const float* py = ym + (size_t)sc * Kc + jc;
        const float* pu = upm + (size_t)sc * Kc + jc;
        const ptrdiff_t step_w = (ptrdiff_t)Sw * C;
        const ptrdiff_t wrap_w = ((ptrdiff_t)Sh * W - (ptrdiff_t)Nw * Sw) * C;
        const ptrdiff_t wrap_h = ((ptrdiff_t)H - (ptrdiff_t)Nh * Sh) * W * C;
        const int n_iter = (s_hi - s_lo + 1) / 2;
        float x0n = px0[0], x1n = px0[second], yn = *py, un = s < s_hi ? *pu : 0.0f;
        for (int it = 0; it < n_iter; ++it) {
            const float x0 = x0n, x1 = x1n, yv = yn, uv = un;
            s += 2;
            if (s < s_hi) {
                py += 2 * Kc; pu += 2 * Kc;
                px0 += 2 * step_w;
                nw += 2;
                while (nw >= Nw) {
                    nw -= Nw; px0 += wrap_w;
                    if (++nh == Nh) { nh = 0; px0 += wrap_h; }
                }
            }
            if (it + 1 < n_iter) {                        // wavefront-uniform
                x0n = px0[0]; x1n = px0[second]; yn = *py;
                un = s < s_hi ? *pu : 0.0f;
            }
            // the inputs of the half's patch, from the lanes that fetched them to all
            __builtin_amdgcn_wave_barrier();
            if ((lane & 16) == 0) {
                xstage[wave][half][l16] = x0;
                xstage[wave][half][l16 + 16] = x1;
            }
            __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
            __builtin_amdgcn_wave_barrier();
            const float ys = yv * -neg_s;
            const float4* __restrict__ xq = reinterpret_cast<const float4*>(xstage[wave][half]);
            auto rows16 = [&](int base) {
                float xr[16];
#pragma unroll
                for (int v = 0; v < 4; ++v) {
                    const float4 x4 = xq[base / 4 + v];
                    xr[4 * v] = x4.x; xr[4 * v + 1] = x4.y; xr[4 * v + 2] = x4.z; xr[4 * v + 3] = x4.w;
                }
#pragma unroll
                for (int r = 0; r < 16; ++r) acc[base + r] = __fmaf_rn(scaled_lead(xr[r], neg_s, ys), uv, acc[base + r]);
            };
            rows16(0);
            if (n_rows > 16) rows16(16);                  // block-uniform
            if (with_bias) acc_bias = __fmaf_rn(scaled_lead(biasvolt, neg_s, ys), uv, acc_bias);
        }
    }
#pragma unroll
    for (int r = 0; r < DWW_RI; ++r) red[wave][r][lane] = acc[r];
    red[wave][DWW_RI][lane] = acc_bias;
    __syncthreads();
    if (wave == 0 && half == 0 && kc < Kc) {
        float* out = dst + (size_t)blockIdx.z * rows * Kc;
#pragma unroll 4
        for (int r = 0; r <= DWW_RI; ++r) {
            if (r == DWW_RI ? !with_bias : r >= n_rows) continue;
            float sum = 0.0f;
#pragma unroll
            for (int wv = 0; wv < 4; ++wv) sum = (sum + red[wv][r][kc]) + red[wv][r][kc + 32];
            out[(size_t)(r == DWW_RI ? bias_row : i0 + r) * Kc + kc] = sum * post;
        }
    }
}

}  // namespace

// Launch shape of the channel-lane dX kernel for a layer (decided by its geometry alone, never by the batch: the
// order of the additions, and with it the last bits of dX, must not depend on the batch size).
struct DxPlan {
    bool ok;
    int parts_shift, span, tiles_w, c_blocks, kcb, ksplit;
    size_t lds;
};
static DxPlan dx_plan(const ConvGeom& g) {
    DxPlan p{};
    if (g.C < 1 || g.Kc % 16 != 0 || g.Nw * g.Kc * 4 >= 0x7fffffffLL) return p;   // (an output row of ym / upm behind one buffer descriptor)
    // Fewer than 32 channels: only with the slot-major sweep of three-column kernels.  The tap-major one pays
    // a few dozen scalar instructions per (pixel, tap) to find the patch, which 16 output channels of 3 or 4
    // input channels do not cover (7x7/2 on 3 channels at 224 x 224, B = 32: 2.8 ms against 2.2 ms through
    // patch space).
    if (g.C < 32 && g.Kw != 3) return p;
    // parts of a wavefront: as many as the channels leave room for, but no wider a tile than the row needs
    int parts = g.C > 32 ? 1 : g.C > 16 ? 2 : g.C > 8 ? 4 : g.C > 4 ? 8 : 16;
    while (parts > 2 && DX_TILE * (parts / 2) >= g.W) parts /= 2;
    p.parts_shift = parts == 1 ? 0 : parts == 2 ? 1 : parts == 4 ? 2 : parts == 8 ? 3 : 4;
    p.span = DX_TILE * parts;
    p.tiles_w = (int)((g.W + p.span - 1) / p.span);
    p.c_blocks = parts > 1 ? 1 : (int)((g.C + kWave - 1) / kWave);
    p.kcb = g.Kc % 64 == 0 ? 64 : (g.Kc % 32 == 0 ? 32 : 16);
    // small images with at least four chunks of output channels: split the channels over the
    // wavefronts of a workgroup.
    // (Up to 1024 tiles per image: with 256 output channels a tile's wavefront walks 36 taps, and at small
    // batches too few tiles exist to hide that -- 256 -> 256 at 16 x 16, one image: 55 against 174 us;
    // at 32 images the split still is a little ahead, 437 against 491 us.)
    // With 128 output channels (two chunks) the split is in two: 64 -> 128 at 28 x 28 is 3840 tiles for 32 images,
    // not quite four per SIMD, and the launch ends on the SIMDs that hold four.
    // Layers with at most 32 input channels and 64 output channels on small images: two chunks of 32.
    const bool few_tiles = g.H * p.tiles_w * p.c_blocks <= 1024;
    if (parts > 1 && few_tiles && g.Kc == 64) p.kcb = 32;
    // the staged rows of a wavefront stay near 12 KB, so that LDS holds them for sixteen wavefronts of a CU
    auto wave_lds = [&](int kcb) { return (size_t)2 * (p.span + g.Kw) * kcb * sizeof(float); };
    while (p.kcb > 16 && wave_lds(p.kcb) > 12 * 1024) p.kcb /= 2;
    p.ksplit = !few_tiles ? 1 : (parts == 1 && g.Kc % (4 * p.kcb) == 0) ? 4 : g.Kc % (2 * p.kcb) == 0 ? 2 : 1;
    auto total_lds = [&]() {
        return p.ksplit * wave_lds(p.kcb) + (p.ksplit > 1 ? (size_t)(p.ksplit - 1) * DX_TILE * kWave * sizeof(float) : 0);
    };
    while (p.ksplit > 1 && total_lds() > 64 * 1024) p.ksplit /= 2;
    p.lds = total_lds();
    p.ok = p.lds <= 64 * 1024;                            // the default limit of a workgroup
    return p;
}

bool cv_grad_input_chan_supported(const ConvGeom& g) { return dx_plan(g).ok; }

// The factor BIG of dx_mac8: the largest power of two with MAX_SPIKE_TIME * BIG <= 2^126.
static float dx_mask_scale(float max_time) {
    int e = 0;
    if (max_time > 1.0f) {
        if (max_time < 0x1p86f) frexpf(max_time, &e);     // max_time < 2^e
        else e = 86;
    }
    return ldexpf(1.0f, 126 - e);
}

// wq: the weights regrouped by launch_backward_prologue (mode 2)
int launch_cv_grad_input_chan(const float* xpad, const float* wq, const float* upm, const float* ym,
                              float* dx, const CropGeom& crop, const ConvGeom& g, const NeuronParams& np,
                              hipStream_t stream) {
    const DxPlan pl = dx_plan(g);
    if (!pl.ok) return fail(SNNTC_ERR_UNSUPPORTED, "conv backward: no channel-lane launch shape for this layer");
    const int span = pl.span, tiles_w = pl.tiles_w, c_blocks = pl.c_blocks, kcb = pl.kcb, ksplit = pl.ksplit;
    const bool multi = pl.parts_shift > 0;
    const int64_t n_items = g.B * g.H * tiles_w * c_blocks;
    // One item per workgroup.  Without the split a workgroup is a single wavefront: the
    // wavefronts do not cooperate, their running times differ (border tiles, rows outside the window),
    // and a CU takes a new workgroup only when a whole one has left, so in larger workgroups the slots
    // of the early finishers would idle.
    const int wg_waves = ksplit;
    // a last tile with at most half its pixels inside the row goes to the end of the launch
    const bool partial_last = tiles_w > 1 && (g.W - (int64_t)(tiles_w - 1) * span) * 2 <= span;
    const int64_t lead_items = partial_last ? g.B * g.H * (tiles_w - 1) * c_blocks : n_items;
    int64_t lead_blocks = lead_items;
    if (partial_last) lead_blocks = (lead_blocks + kXcds - 1) / kXcds * kXcds;
    const int64_t blocks = lead_blocks + (n_items - lead_items);
    if (blocks > 0x7fffffffLL) return fail(SNNTC_ERR_TOO_LARGE, "conv backward: grid too large");
    dim3 grid((unsigned)blocks), block(wg_waves * kWave);
    const size_t lds = pl.lds;
    void (*kern)(const float*, const float*, const float*, const float*, float*, CropGeom, int, int, int, int, int, int,
                 int, int, int, int, int, int, int64_t, int64_t, int, float, int, float, int);
    if (g.Kw == 3) {
        if (multi)
            kern = kcb == 64 ? cv_grad_input_chan_kernel<64, true, 3> : kcb == 32 ? cv_grad_input_chan_kernel<32, true, 3>
                                                                                   : cv_grad_input_chan_kernel<16, true, 3>;
        else
            kern = kcb == 64 ? cv_grad_input_chan_kernel<64, false, 3> : kcb == 32 ? cv_grad_input_chan_kernel<32, false, 3>
                                                                                    : cv_grad_input_chan_kernel<16, false, 3>;
    } else if (multi) {
        kern = kcb == 64 ? cv_grad_input_chan_kernel<64, true, 0> : kcb == 32 ? cv_grad_input_chan_kernel<32, true, 0>
                                                                               : cv_grad_input_chan_kernel<16, true, 0>;
    } else {
        kern = kcb == 64 ? cv_grad_input_chan_kernel<64, false, 0> : kcb == 32 ? cv_grad_input_chan_kernel<32, false, 0>
                                                                                : cv_grad_input_chan_kernel<16, false, 0>;
    }
    {
        KernelTimerScope timer_("cv_grad_input", stream);
        hipLaunchKernelGGL(kern, grid, block, lds, stream, xpad, wq, upm, ym, dx, crop, (int)g.H, (int)g.W, (int)g.C,
                           (int)g.Kc, (int)g.Kh, (int)g.Kw, (int)g.Sh, (int)g.Sw, (int)g.Nh, (int)g.Nw, tiles_w,
                           c_blocks, n_items, lead_items, (int)lead_blocks, np.max_cmp, ksplit, dx_mask_scale(np.max_time),
                           pl.parts_shift);
    }
    SNNTC_HIP_CHECK(hipGetLastError());
    return SNNTC_OK;
}

// Any channel count; with very short kernel rows (Kw*C < 9) a block would mostly carry unused rows.
bool cv_grad_weight_wide_supported(const ConvGeom& g) { return g.Kw * g.C >= 9; }

static int64_t cv_grad_weight_row_blocks(const ConvGeom& g) {
    return g.Kh * ((g.Kw * g.C + DWW_RI - 1) / DWW_RI);
}

int cv_grad_weight_wide_blocks(const ConvGeom& g) {
    return (int)(((g.Kc + kWave - 1) / kWave) * cv_grad_weight_row_blocks(g));
}

// All rows of dW, bias row included (or of every partial-sum slice when nsplit > 1).
int launch_cv_grad_weight_wide(const float* xpad, const float* upm, const float* ym, float* dst, int nsplit,
                               const ConvGeom& g, int64_t rows, const NeuronParams& np, hipStream_t stream) {
    const int seg_per_slice = (int)((g.S + nsplit - 1) / nsplit);
    dim3 grid((unsigned)((g.Kc + kWave - 1) / kWave), (unsigned)cv_grad_weight_row_blocks(g), (unsigned)nsplit);
    if (grid.y > 65535u) return fail(SNNTC_ERR_TOO_LARGE, "weight gradient: too many weight rows");
    // patches before s_safe can fetch DWW_RI floats from any of their kernel-row starts without leaving
    // the image tensor (only the last few patches of the last image cannot)
    const int64_t n_x = g.B * g.H * g.W * g.C;
    int64_t s_safe = g.S;
    while (s_safe > 0) {
        const int64_t sp = s_safe - 1, per_img = g.Nh * g.Nw;
        const int64_t a = sp / per_img, nh = (sp % per_img) / g.Nw, nw = sp % g.Nw;
        const int64_t last_start = ((a * g.H + nh * g.Sh + g.Kh - 1) * g.W + nw * g.Sw) * g.C + g.Kw * g.C - 1;
        if (last_start + DWW_RI <= n_x) break;
        --s_safe;
    }
    {
        KernelTimerScope timer_("grad_weight", stream);
        const bool full = (g.Kw * g.C) % DWW_RI == 0;
        const LeadScale ls = lead_scale(np.max_time);
        // layers whose kernel rows are shorter than a block: work on the multiple of 8 rows above Kw*C
        const int64_t kwc = g.Kw * g.C;
        auto wide = full ? cv_grad_weight_wide_kernel<true, DWW_RI> : cv_grad_weight_wide_kernel<false, DWW_RI>;
        if (kwc <= 8) wide = cv_grad_weight_wide_kernel<false, 8>;
        else if (kwc <= 16) wide = cv_grad_weight_wide_kernel<false, 16>;
        else if (kwc <= 24) wide = cv_grad_weight_wide_kernel<false, 24>;
        hipLaunchKernelGGL(g.Kc <= 32 ? cv_grad_weight_narrow_kernel : wide, grid, dim3(256), 0,
                           stream, xpad, upm, ym, dst, (int)g.S, (int)g.Kc, (int)rows, seg_per_slice, (int)g.H,
                           (int)g.W, (int)g.C, (int)g.Kw, (int)g.Sh, (int)g.Sw, (int)g.Nh, (int)g.Nw,
                           np.bias ? (int)g.P : -1, np.biasvolt, (int)s_safe, ls.neg_s, ls.post);
    }
    SNNTC_HIP_CHECK(hipGetLastError());
    return SNNTC_OK;
}

}  // namespace snntc
