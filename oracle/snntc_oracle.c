/*
 * snntc_oracle.c -- CPU restatement of the SNN-TC custom ops.  TEST INFRASTRUCTURE ONLY.
 *
 * This file is the checker for the HIP library, never the product: only the test-suite, the
 * smoke check and the benchmark's cpu_baseline leg may link or call it.  Nothing under the
 * shipped package may depend on it.
 *
 * Two families of functions live here, both following the reference sources cited next to
 * each function (paths relative to the reference checkout):
 *
 *   *_dev  "device semantics": what the reference's GPU kernels compute (these define the
 *          op contract: bias processed first, scan stops at inputs > MAX-0.1, division-free
 *          firing test, second output half = 1/(sum w - theta), gradient mask x <= y).
 *          The sort is a STABLE ascending sort (ties by ascending index); the reference's
 *          cub::DeviceSegmentedSort leaves tie order unspecified, so stable order is the
 *          one deterministic member of the set of orders the reference may produce.
 *          Accumulation is sequential fp32 with fused multiply-add exactly where the device
 *          compiler fuses (`ysum += x*w`, `accu += a*b`), and the reciprocal is an exactly
 *          rounded 1/wsum (the reference's __fdividef is a ~2 ulp approximation of it).
 *
 *   *_host "host semantics": what the reference's single-threaded CPU functors compute,
 *          including their documented limitations (second half holds wsum, strict x < y
 *          gradient mask, no bias in the dense backward, the dense-forward bias `break`).
 *          These are the timed CPU baseline and a structurally different cross-check.
 *
 * Parity pinning status (see tests/test_oracle_*.py): every function here is pinned by the
 * reference-held closed form (test-snn-fc-forward.py:83-89, test-snn-cv-forward.py:126-146),
 * by brute-force/independent restatements, by invariants, and -- for gradients -- by central
 * finite differences of a float64 forward.  Tie order inside the reference's GPU sort is
 * implementation-defined in the reference itself and therefore "parity unpinned".
 *
 * Build: see oracle/Makefile (gcc -O3 -ffp-contract=off -mfma).
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define SNNTC_EXPORT __attribute__((visibility("default")))

/* ------------------------------------------------------------------------------------------
 * Stable ascending argsort of one segment (bottom-up merge, ties keep the lower index first).
 * Follows the behaviour of BottomUpMergeSort, snntc/snnfc_kernels.cc:17-70: a merge that takes
 * the left run's head when it is <= the right run's head, started from the identity index
 * array.  `keys` is overwritten with the sorted keys, `perm` receives the source indices.
 * ---------------------------------------------------------------------------------------- */
static void stable_argsort(float* keys, int32_t* perm, int n, float* tk, int32_t* tp) {
    for (int i = 0; i < n; ++i) perm[i] = i;
    float* ak = keys; int32_t* ap = perm;
    float* bk = tk;   int32_t* bp = tp;
    for (int run = 1; run < n; run *= 2) {
        for (int lo = 0; lo < n; lo += 2 * run) {
            int mid = lo + run < n ? lo + run : n;
            int hi = lo + 2 * run < n ? lo + 2 * run : n;
            int l = lo, r = mid;
            for (int o = lo; o < hi; ++o) {
                int take_left = (l < mid) && (r >= hi || ak[l] <= ak[r]);
                if (take_left) { bk[o] = ak[l]; bp[o] = ap[l]; ++l; }
                else           { bk[o] = ak[r]; bp[o] = ap[r]; ++r; }
            }
        }
        float* sk = ak; ak = bk; bk = sk;
        int32_t* sp = ap; ap = bp; bp = sp;
    }
    if (ak != keys) {
        memcpy(keys, ak, (size_t)n * sizeof(float));
        memcpy(perm, ap, (size_t)n * sizeof(int32_t));
    }
}

/* Segmented stable sort of a [S, I] matrix: sorted[s,:] ascending, perm[s,:] source columns. */
SNNTC_EXPORT int snntc_oracle_sort_segments(const float* x, int64_t S, int64_t I,
                                            float* sorted, int32_t* perm) {
    float* tk = (float*)malloc((size_t)(I > 0 ? I : 1) * sizeof(float));
    int32_t* tp = (int32_t*)malloc((size_t)(I > 0 ? I : 1) * sizeof(int32_t));
    if (!tk || !tp) { free(tk); free(tp); return 1; }
    for (int64_t s = 0; s < S; ++s) {
        memcpy(sorted + s * I, x + s * I, (size_t)I * sizeof(float));
        stable_argsort(sorted + s * I, perm + s * I, (int)I, tk, tp);
    }
    free(tk); free(tp);
    return 0;
}

/* ------------------------------------------------------------------------------------------
 * Causal-set scan of one (segment, output) pair, device semantics.
 * Follows SnnFcCudaOutKernel, snntc/snnfc_kernels.cu.cc:25-70 (identical to
 * SnnFcCudaOutKernelBias, snntc/snncv_kernels.cu.cc:19-72).
 *   xs/perm : the segment sorted ascending and its permutation
 *   w       : weight matrix [I + bias, J] row-major, column j is scanned
 * Returns the number of sorted inputs consumed; *y and *rcp get the two output halves.
 * *fired_out tells whether the neuron fired (consumed count alone cannot tell).
 * ---------------------------------------------------------------------------------------- */
static int scan_dev(const float* xs, const int32_t* perm, const float* w, int64_t I, int64_t J,
                    int64_t j, float max_time, float theta, float biasvolt,
                    float* y, float* rcp, int* fired_out) {
    const float max_cmp = max_time - 0.1f;
    float wsum = -theta, ysum = 0.0f, wa = 0.0f, ya = 0.0f;
    int fired = 0;
    if (biasvolt > 1e-8f) {
        float wb = w[I * J + j];
        wsum += wb;
        ysum = biasvolt * wb;
        wa = wsum; ya = ysum;
        if (wa < 0.0f) { wa = -wa; ya = -ya; }
        fired = ya > wa * biasvolt;
    }
    int k = 0;
    for (; k < I; ++k) {
        float x = xs[k];
        if (x > max_cmp) break;
        if (fired && ya <= x * wa) break;
        float wk = w[(int64_t)perm[k] * J + j];
        wsum += wk;
        ysum = fmaf(x, wk, ysum);
        wa = wsum; ya = ysum;
        if (wa < 0.0f) { wa = -wa; ya = -ya; }
        fired = ya > x * wa;
    }
    float out = max_time, r = 0.0f;
    if (fired) {
        r = 1.0f / wsum;
        out = ysum * r;
        if (out >= max_time) { out = max_time; r = 0.0f; }
    }
    *y = out; *rcp = r; *fired_out = fired;
    return k;
}

/* Dense forward, device semantics.  x[B,I], w[I+bias,J], params[6] as built by SNN_dense
 * (SNN_TC_Modules.py:48-49): {MAX, eps, theta, tpb, blocks, biasvolt}.
 * out[2B,J]: rows [0,B) spike times, rows [B,2B) 1/(sum w - theta) (0 when not fired).
 * Optional: causal_k[B,J] (consumed inputs, -1 when not fired), sorted[B,I], perm[B,I].
 * Follows SnnFcFunctor<GPUDevice>, snntc/snnfc_kernels.cu.cc:93-194. */
SNNTC_EXPORT int snntc_oracle_fc_forward_dev(const float* x, const float* w, const float* params,
                                             float* out, int32_t* causal_k, float* sorted_out,
                                             int32_t* perm_out, int64_t B, int64_t I, int64_t J) {
    const float max_time = params[0], theta = params[2], biasvolt = params[5];
    size_t n = (size_t)(B * I > 0 ? B * I : 1);
    float* sorted = sorted_out ? sorted_out : (float*)malloc(n * sizeof(float));
    int32_t* perm = perm_out ? perm_out : (int32_t*)malloc(n * sizeof(int32_t));
    if (!sorted || !perm) return 1;
    int rc = snntc_oracle_sort_segments(x, B, I, sorted, perm);
    if (rc == 0) {
        for (int64_t b = 0; b < B; ++b) {
            for (int64_t j = 0; j < J; ++j) {
                float y, r; int fired;
                int k = scan_dev(sorted + b * I, perm + b * I, w, I, J, j, max_time, theta,
                                 biasvolt, &y, &r, &fired);
                out[b * J + j] = y;
                out[(B + b) * J + j] = r;
                if (causal_k) causal_k[b * J + j] = (fired && r != 0.0f) ? k : -1;
            }
        }
    }
    if (!sorted_out) free(sorted);
    if (!perm_out) free(perm);
    return rc;
}

/* Dense forward, host semantics: SnnFcFunctor<CPUDevice>, snntc/snnfc_kernels.cc:75-151.
 * Second half of out holds (sum w - theta) itself, not its reciprocal.  Products and sums are
 * rounded separately (the reference CPU build has no FMA contraction).  The bias block's
 * `break` leaves the loop over outputs of that sample, as the reference does. */
SNNTC_EXPORT int snntc_oracle_fc_forward_host(const float* x, const float* w, const float* params,
                                              float* out, int64_t B, int64_t I, int64_t J) {
    const float max_time = params[0], eps = params[1], theta = params[2], biasvolt = params[5];
    size_t n = (size_t)(B * I > 0 ? B * I : 1);
    float* sorted = (float*)malloc(n * sizeof(float));
    int32_t* perm = (int32_t*)malloc(n * sizeof(int32_t));
    if (!sorted || !perm) { free(sorted); free(perm); return 1; }
    snntc_oracle_sort_segments(x, B, I, sorted, perm);
    const int64_t half = B * J;
    for (int64_t t = 0; t < half; ++t) { out[t] = max_time; out[half + t] = 0.0f; }
    for (int64_t b = 0; b < B; ++b) {
        const float* xr = x + b * I;
        const int32_t* pr = perm + b * I;
        for (int64_t j = 0; j < J; ++j) {
            float prod;   /* products rounded separately: build with -ffp-contract=off */
            float wsum = -theta, ysum = 0.0f;
            if (biasvolt > 1e-8f) {
                float wb = w[I * J + j];
                wsum += wb;
                prod = biasvolt * wb; ysum += prod;
                if (wsum > eps || wsum < -eps) {
                    float cand = ysum / wsum;
                    if (cand > biasvolt && I > 0 && cand <= xr[pr[0]]) {
                        out[b * J + j] = cand; out[half + b * J + j] = wsum;
                        break;                      /* reference: exits the j loop */
                    }
                }
            }
            for (int64_t i = 0; i < I; ++i) {
                float xi = xr[pr[i]];
                float wi = w[(int64_t)pr[i] * J + j];
                wsum = wsum + wi;
                prod = xi * wi; ysum = ysum + prod;
                if (wsum < eps && wsum > -eps) continue;
                float cand = ysum / wsum;
                if (cand > xi) {
                    if (i < I - 1) {
                        if (cand <= xr[pr[i + 1]]) {
                            out[b * J + j] = cand; out[half + b * J + j] = wsum;
                            break;
                        }
                    } else if (cand < max_time) {
                        out[b * J + j] = cand; out[half + b * J + j] = wsum;
                    }
                }
            }
        }
    }
    free(sorted); free(perm);
    return 0;
}

/* ------------------------------------------------------------------------------------------
 * Dense backward, device semantics.  grad[2B,J] (only rows [0,B) are used), oldout[2B,J].
 *   up = grad[:B] * oldout[B:]                        snntc/snnfcgrad_kernels.cu.cc:159-173
 *   dX : SnnFcGradCudaKernelInput                     snntc/snnfcgrad_kernels.cu.cc:15-71
 *   dW : SnnFcGradCudaKernelWeight (bias row uses x = biasvolt)          ...:74-133
 * Sequential fp32 accumulation (fused multiply-add) in ascending j (dX) / ascending b (dW),
 * which is the order the reference's tile loops visit the terms.  With wide != 0 the sums are
 * carried in double instead (used by the tests to bound re-association error).
 * dparams[6] is written with zeros (the reference GPU leaves it unwritten).
 * ---------------------------------------------------------------------------------------- */
SNNTC_EXPORT int snntc_oracle_fc_backward_dev(const float* grad, const float* x, const float* w,
                                              const float* params, const float* oldout,
                                              float* dx, float* dw, float* dparams,
                                              int64_t B, int64_t I, int64_t J, int wide) {
    const float max_cmp = params[0] - 0.1f, biasvolt = params[5];
    const int bias = biasvolt > 1e-8f;
    float* up = (float*)malloc((size_t)(B * J > 0 ? B * J : 1) * sizeof(float));
    if (!up) return 1;
    for (int64_t t = 0; t < B * J; ++t) up[t] = grad[t] * oldout[B * J + t];
    for (int64_t b = 0; b < B; ++b) {
        for (int64_t i = 0; i < I; ++i) {
            const float xv = x[b * I + i];
            float acc = 0.0f; double accd = 0.0;
            for (int64_t j = 0; j < J; ++j) {
                const float yv = oldout[b * J + j];
                if (xv > yv || yv > max_cmp) continue;
                if (wide) accd += (double)up[b * J + j] * (double)w[i * J + j];
                else acc = fmaf(up[b * J + j], w[i * J + j], acc);
            }
            dx[b * I + i] = wide ? (float)accd : acc;
        }
    }
    for (int64_t i = 0; i < I + bias; ++i) {
        for (int64_t j = 0; j < J; ++j) {
            float acc = 0.0f; double accd = 0.0;
            for (int64_t b = 0; b < B; ++b) {
                const float xv = (i < I) ? x[b * I + i] : biasvolt;
                const float yv = oldout[b * J + j];
                if (xv > max_cmp || yv > max_cmp || xv > yv) continue;
                if (wide) accd += ((double)xv - (double)yv) * (double)up[b * J + j];
                else acc = fmaf(xv - yv, up[b * J + j], acc);
            }
            dw[i * J + j] = wide ? (float)accd : acc;
        }
    }
    if (dparams) for (int t = 0; t < 6; ++t) dparams[t] = 0.0f;
    free(up);
    return 0;
}

/* Dense backward, host semantics: SnnFcGradFunctor<CPUDevice>, snntc/snnfcgrad_kernels.cc:17-84.
 * Recomputes wsum from the strict mask x < y without the bias weight, divides by it, never
 * writes a bias row of dW (rows >= I are left untouched), zeroes dparams[0..4]. */
SNNTC_EXPORT int snntc_oracle_fc_backward_host(const float* grad, const float* x, const float* w,
                                               const float* params, const float* oldout,
                                               float* dx, float* dw, float* dparams,
                                               int64_t B, int64_t I, int64_t J) {
    const float max_time = params[0], theta = params[2];
    const double max_cmp = (double)max_time - 0.1;   /* the reference compares in double */
    float* wsum = (float*)malloc((size_t)(B * J > 0 ? B * J : 1) * sizeof(float));
    if (!wsum) return 1;
    float prod;
    if (dparams) for (int t = 0; t <= 4; ++t) dparams[t] = 0.0f;
    for (int64_t b = 0; b < B; ++b)
        for (int64_t j = 0; j < J; ++j) {
            const int64_t k = b * J + j;
            if (oldout[k] > max_cmp) { wsum[k] = max_time; continue; }
            float s = -theta;
            for (int64_t i = 0; i < I; ++i)
                if (x[b * I + i] < oldout[k]) s += w[i * J + j];
            wsum[k] = s;
        }
    for (int64_t b = 0; b < B; ++b)
        for (int64_t i = 0; i < I; ++i) {
            float acc = 0.0f;
            for (int64_t j = 0; j < J; ++j) {
                const int64_t k = b * J + j;
                if (x[b * I + i] < oldout[k] && oldout[k] < max_cmp) {
                    prod = grad[k] * w[i * J + j];
                    prod = prod / wsum[k];
                    acc += prod;
                }
            }
            dx[b * I + i] = acc;
        }
    for (int64_t i = 0; i < I; ++i)
        for (int64_t j = 0; j < J; ++j) {
            float acc = 0.0f;
            for (int64_t b = 0; b < B; ++b) {
                const int64_t k = b * J + j;
                const float xv = x[b * I + i];
                if (xv < oldout[k] && oldout[k] < max_cmp) {
                    prod = xv - oldout[k];
                    prod = grad[k] * prod;
                    prod = prod / wsum[k];
                    acc += prod;
                }
            }
            dw[i * J + j] = acc;
        }
    free(wsum);
    return 0;
}

/* ------------------------------------------------------------------------------------------
 * Convolution helpers.  xpad[B,H,W,C] is the already padded/cropped NHWC input, the op derives
 * Nh=(H-Kh)/Sh+1, Nw=(W-Kw)/Sw+1 (snntc/snncv_kernels.cc:215).  A patch is indexed
 * s=(a*Nh+nh)*Nw+nw and its elements i=(kh*Kw+kw)*C+c (snntc/snncvgrad_kernels.cu.cc:39-41).
 * params[12] as built by SNN_conv (SNN_TC_Modules.py:121-123):
 *   {MAX, tpb, blocks, eps, theta, cudaflag, Kh, Kw, Sh, Sw, same, biasvolt}.
 * ---------------------------------------------------------------------------------------- */
typedef struct { int64_t B, H, W, C, Kc, Kh, Kw, Sh, Sw, Nh, Nw, P, S; } cv_geom;

static cv_geom make_geom(const float* params, int64_t B, int64_t H, int64_t W, int64_t C,
                         int64_t Kc) {
    cv_geom g;
    g.B = B; g.H = H; g.W = W; g.C = C; g.Kc = Kc;
    g.Kh = (int64_t)params[6]; g.Kw = (int64_t)params[7];
    g.Sh = (int64_t)params[8]; g.Sw = (int64_t)params[9];
    g.Nh = (H - g.Kh) / g.Sh + 1; g.Nw = (W - g.Kw) / g.Sw + 1;
    g.P = g.Kh * g.Kw * C; g.S = B * g.Nh * g.Nw;
    return g;
}

/* im2col: patches[S,P] from xpad, VALID, depth order (kh,kw,c).  Layout as produced by the
 * reference's extract_image_patches call, snntc/snncv_kernels.cu.cc:112-120. */
SNNTC_EXPORT int snntc_oracle_im2col(const float* xpad, const float* params, float* patches,
                                     int64_t B, int64_t H, int64_t W, int64_t C) {
    cv_geom g = make_geom(params, B, H, W, C, 1);
    for (int64_t a = 0; a < B; ++a)
        for (int64_t nh = 0; nh < g.Nh; ++nh)
            for (int64_t nw = 0; nw < g.Nw; ++nw) {
                float* dst = patches + ((a * g.Nh + nh) * g.Nw + nw) * g.P;
                for (int64_t kh = 0; kh < g.Kh; ++kh)
                    for (int64_t kw = 0; kw < g.Kw; ++kw)
                        memcpy(dst + (kh * g.Kw + kw) * C,
                               xpad + ((a * H + nh * g.Sh + kh) * W + nw * g.Sw + kw) * C,
                               (size_t)C * sizeof(float));
            }
    return 0;
}

/* Conv forward, device semantics: im2col, per-patch stable sort, the same scan as the dense op
 * (SnnCvFunctor<GPUDevice>, snntc/snncv_kernels.cu.cc:95-210).  out[2B,Nh,Nw,Kc]. */
SNNTC_EXPORT int snntc_oracle_cv_forward_dev(const float* xpad, const float* w, const float* params,
                                             float* out, int32_t* causal_k, float* sorted_out,
                                             int32_t* perm_out, int64_t B, int64_t H, int64_t W,
                                             int64_t C, int64_t Kc) {
    cv_geom g = make_geom(params, B, H, W, C, Kc);
    float* patches = (float*)malloc((size_t)(g.S * g.P > 0 ? g.S * g.P : 1) * sizeof(float));
    if (!patches) return 1;
    snntc_oracle_im2col(xpad, params, patches, B, H, W, C);
    float p6[6] = { params[0], params[3], params[4], 0.0f, 0.0f, params[11] };
    int rc = snntc_oracle_fc_forward_dev(patches, w, p6, out, causal_k, sorted_out, perm_out,
                                         g.S, g.P, Kc);
    free(patches);
    return rc;
}

/* Conv forward, host semantics: SnnCvFunctor<CPUDevice>, snntc/snncv_kernels.cc:75-183.
 * One stable sort of the whole padded sample, then an event-driven pass: inputs are visited in
 * ascending order and pushed into every output whose window covers them; each output keeps a
 * running (ysum, wsum, candidate, count) and locks once its candidate precedes the next input.
 * Writes only out[0 : B*Nh*Nw*Kc] (the reference never writes the second half). */
SNNTC_EXPORT int snntc_oracle_cv_forward_host(const float* xpad, const float* w, const float* params,
                                              float* out, int64_t B, int64_t H, int64_t W,
                                              int64_t C, int64_t Kc) {
    cv_geom g = make_geom(params, B, H, W, C, Kc);
    const float max_time = params[0], eps = params[3], theta = params[4];
    const int bias = params[11] > 1e-8f;
    const float xbias = bias ? params[11] : 1.0f;
    const int64_t n_in = H * W * C, n_out = g.Nh * g.Nw * Kc;
    float* keys = (float*)malloc((size_t)n_in * sizeof(float));
    float* tk = (float*)malloc((size_t)n_in * sizeof(float));
    int32_t* order = (int32_t*)malloc((size_t)n_in * sizeof(int32_t));
    int32_t* tp = (int32_t*)malloc((size_t)n_in * sizeof(int32_t));
    int32_t* cnt = (int32_t*)malloc((size_t)n_out * sizeof(int32_t));
    float* ys = (float*)malloc((size_t)n_out * sizeof(float));
    float* ws = (float*)malloc((size_t)n_out * sizeof(float));
    if (!keys || !tk || !order || !tp || !cnt || !ys || !ws) return 1;
    float prod;
    const int32_t UNSEEN = -1000000000;
    for (int64_t a = 0; a < B; ++a) {
        const float* xin = xpad + a * n_in;
        float* o = out + a * n_out;
        memcpy(keys, xin, (size_t)n_in * sizeof(float));
        stable_argsort(keys, order, (int)n_in, tk, tp);
        for (int64_t e = 0; e < n_out; ++e) {
            const int64_t kc = e % Kc;
            float wsum, ysum;
            if (bias) { wsum = w[g.P * Kc + kc] - theta; prod = xbias * w[g.P * Kc + kc]; ysum = prod; }
            else      { wsum = -theta; ysum = 0.0f; }
            cnt[e] = UNSEEN;
            float cand = (wsum != 0.0f) ? ysum / wsum : ysum / eps;
            ys[e] = ysum; ws[e] = wsum;
            o[e] = (cand > xbias && cand < max_time) ? cand : max_time * 10.0f;
        }
        for (int64_t t = 0; t < n_in; ++t) {
            const int64_t src = order[t];
            const int64_t ih = src / (W * C), iw = (src % (W * C)) / C, ic = src % C;
            const float v = xin[src];
            int64_t nh0 = (int64_t)ceil((double)(ih - g.Kh + 1) / (double)g.Sh); if (nh0 < 0) nh0 = 0;
            int64_t nh1 = ih / g.Sh; if (nh1 > g.Nh - 1) nh1 = g.Nh - 1;
            int64_t nw0 = (int64_t)ceil((double)(iw - g.Kw + 1) / (double)g.Sw); if (nw0 < 0) nw0 = 0;
            int64_t nw1 = iw / g.Sw; if (nw1 > g.Nw - 1) nw1 = g.Nw - 1;
            for (int64_t nh = nh0; nh <= nh1; ++nh)
                for (int64_t nw = nw0; nw <= nw1; ++nw) {
                    const int64_t wrow = ((ih - nh * g.Sh) * g.Kw + (iw - nw * g.Sw)) * C + ic;
                    for (int64_t kc = 0; kc < Kc; ++kc) {
                        const int64_t e = (nh * g.Nw + nw) * Kc + kc;
                        int32_t k = cnt[e];
                        if (k >= 0) continue;                 /* locked: already fired */
                        if (k < -100000000) { cnt[e] = 0; k = 0; }
                        if (o[e] <= v) { cnt[e] = -k; continue; }   /* candidate precedes v */
                        if ((double)v >= (double)max_time - 1.0) continue;   /* padding never contributes */
                        float wsum = ws[e], ysum = ys[e];
                        const float wt = w[wrow * Kc + kc];
                        wsum = wsum + wt;
                        prod = v * wt; ysum = ysum + prod;
                        float cand = (wsum < eps && wsum > -eps) ? ysum / eps : ysum / wsum;
                        o[e] = (cand > v) ? cand : max_time * 10.0f;
                        ys[e] = ysum; ws[e] = wsum;
                        cnt[e] -= 1;
                    }
                }
        }
        for (int64_t e = 0; e < n_out; ++e)
            if (cnt[e] < 0 && !(o[e] < max_time)) o[e] = max_time;
    }
    free(keys); free(tk); free(order); free(tp); free(cnt); free(ys); free(ws);
    return 0;
}

/* Conv backward, device semantics.  grad/oldout [2B,Nh,Nw,Kc]; dxpad[B,H,W,C]; dw[P+bias,Kc].
 *   up   : snntc/snncvgrad_kernels.cu.cc:190-204
 *   dX   : SnnCvGradCudaKernelInput (...:15-84): per (patch, element) sum over kc, then added
 *          into dxpad.  The reference adds with atomicAdd in an unspecified order; here the
 *          additions happen in ascending (patch, element) order.
 *   dW   : SnnCvGradCudaKernelWeightBias (...:90-161), ascending patch order.
 * wide != 0 carries every sum in double. */
SNNTC_EXPORT int snntc_oracle_cv_backward_dev(const float* grad, const float* xpad, const float* w,
                                              const float* params, const float* oldout,
                                              float* dxpad, float* dw, float* dparams,
                                              int64_t B, int64_t H, int64_t W, int64_t C,
                                              int64_t Kc, int wide) {
    cv_geom g = make_geom(params, B, H, W, C, Kc);
    const float max_cmp = params[0] - 0.1f, biasvolt = params[11];
    const int bias = biasvolt > 1e-8f;
    const int64_t SJ = g.S * Kc;
    float* up = (float*)malloc((size_t)(SJ > 0 ? SJ : 1) * sizeof(float));
    double* dxd = wide ? (double*)calloc((size_t)(B * H * W * C > 0 ? B * H * W * C : 1), sizeof(double)) : NULL;
    if (!up || (wide && !dxd)) return 1;
    for (int64_t t = 0; t < SJ; ++t) up[t] = grad[t] * oldout[SJ + t];
    for (int64_t t = 0; t < B * H * W * C; ++t) dxpad[t] = 0.0f;
    for (int64_t s = 0; s < g.S; ++s) {
        const int64_t a = s / (g.Nh * g.Nw), nh = (s % (g.Nh * g.Nw)) / g.Nw, nw = s % g.Nw;
        for (int64_t i = 0; i < g.P; ++i) {
            const int64_t kh = i / (g.Kw * C), kw = (i % (g.Kw * C)) / C, c = i % C;
            const int64_t src = ((a * H + nh * g.Sh + kh) * W + nw * g.Sw + kw) * C + c;
            const float xv = xpad[src];
            float acc = 0.0f; double accd = 0.0;
            for (int64_t j = 0; j < Kc; ++j) {
                const float yv = oldout[s * Kc + j];
                if (xv > yv || yv > max_cmp) continue;
                if (wide) accd += (double)up[s * Kc + j] * (double)w[i * Kc + j];
                else acc = fmaf(up[s * Kc + j], w[i * Kc + j], acc);
            }
            if (wide) dxd[src] += accd; else dxpad[src] += acc;
        }
    }
    if (wide) for (int64_t t = 0; t < B * H * W * C; ++t) dxpad[t] = (float)dxd[t];
    for (int64_t i = 0; i < g.P + bias; ++i) {
        const int64_t kh = i / (g.Kw * C), kw = (i % (g.Kw * C)) / C, c = i % C;
        for (int64_t j = 0; j < Kc; ++j) {
            float acc = 0.0f; double accd = 0.0;
            for (int64_t s = 0; s < g.S; ++s) {
                const int64_t a = s / (g.Nh * g.Nw), nh = (s % (g.Nh * g.Nw)) / g.Nw, nw = s % g.Nw;
                const float xv = (i < g.P)
                    ? xpad[((a * H + nh * g.Sh + kh) * W + nw * g.Sw + kw) * C + c] : biasvolt;
                const float yv = oldout[s * Kc + j];
                if (xv > max_cmp || yv > max_cmp || xv > yv) continue;
                if (wide) accd += ((double)xv - (double)yv) * (double)up[s * Kc + j];
                else acc = fmaf(xv - yv, up[s * Kc + j], acc);
            }
            dw[i * Kc + j] = wide ? (float)accd : acc;
        }
    }
    if (dparams) for (int t = 0; t < 12; ++t) dparams[t] = 0.0f;
    free(up); free(dxd);
    return 0;
}

/* Conv backward, host semantics: SnnCvGradFunctor<CPUDevice>, snntc/snncvgrad_kernels.cc:16-122.
 * wsum recomputed from the strict mask (bias weight included), gather-form dX that skips padded
 * inputs, dW including the bias row, dparams[0..9] zeroed.  Uses grad[0:S*Kc] directly (the host
 * functor never multiplies by the stored second half). */
SNNTC_EXPORT int snntc_oracle_cv_backward_host(const float* grad, const float* xpad, const float* w,
                                               const float* params, const float* oldout,
                                               float* dxpad, float* dw, float* dparams,
                                               int64_t B, int64_t H, int64_t W, int64_t C,
                                               int64_t Kc) {
    cv_geom g = make_geom(params, B, H, W, C, Kc);
    const float max_time = params[0], theta = params[4];
    const double max_cmp = (double)max_time - 0.1;   /* the reference compares in double */
    const int bias = params[11] > 1e-8f;
    const float xbias = bias ? params[11] : 1.0f;
    const int64_t SJ = g.S * Kc;
    float* wsum = (float*)malloc((size_t)(SJ > 0 ? SJ : 1) * sizeof(float));
    if (!wsum) return 1;
    float prod;
    if (dparams) for (int t = 0; t < 10; ++t) dparams[t] = 0.0f;
    for (int64_t s = 0; s < g.S; ++s) {
        const int64_t a = s / (g.Nh * g.Nw), nh = (s % (g.Nh * g.Nw)) / g.Nw, nw = s % g.Nw;
        for (int64_t kc = 0; kc < Kc; ++kc) {
            const int64_t k = s * Kc + kc;
            if (!(oldout[k] < max_cmp)) { wsum[k] = max_time; continue; }
            float acc = bias ? w[g.P * Kc + kc] - theta : -theta;
            for (int64_t kh = 0; kh < g.Kh; ++kh)
                for (int64_t kw = 0; kw < g.Kw; ++kw)
                    for (int64_t c = 0; c < C; ++c)
                        if (xpad[((a * H + nh * g.Sh + kh) * W + nw * g.Sw + kw) * C + c] < oldout[k])
                            acc += w[((kh * g.Kw + kw) * C + c) * Kc + kc];
            wsum[k] = acc;
        }
    }
    for (int64_t a = 0; a < B; ++a)
        for (int64_t h = 0; h < H; ++h)
            for (int64_t x = 0; x < W; ++x)
                for (int64_t c = 0; c < C; ++c) {
                    const int64_t src = ((a * H + h) * W + x) * C + c;
                    const float v = xpad[src];
                    dxpad[src] = 0.0f;
                    if (v > max_cmp) continue;
                    int64_t nh0 = (int64_t)ceil((double)(h - g.Kh + 1) / (double)g.Sh); if (nh0 < 0) nh0 = 0;
                    int64_t nh1 = h / g.Sh; if (nh1 > g.Nh - 1) nh1 = g.Nh - 1;
                    int64_t nw0 = (int64_t)ceil((double)(x - g.Kw + 1) / (double)g.Sw); if (nw0 < 0) nw0 = 0;
                    int64_t nw1 = x / g.Sw; if (nw1 > g.Nw - 1) nw1 = g.Nw - 1;
                    float acc = 0.0f;
                    for (int64_t nh = nh0; nh <= nh1; ++nh)
                        for (int64_t nw = nw0; nw <= nw1; ++nw) {
                            const int64_t wrow = ((h - nh * g.Sh) * g.Kw + (x - nw * g.Sw)) * C + c;
                            const int64_t k0 = ((a * g.Nh + nh) * g.Nw + nw) * Kc;
                            for (int64_t kc = 0; kc < Kc; ++kc)
                                if (v < oldout[k0 + kc] && oldout[k0 + kc] < max_cmp) {
                                    prod = grad[k0 + kc] * w[wrow * Kc + kc];
                                    prod = prod / wsum[k0 + kc];
                                    acc += prod;
                                }
                        }
                    dxpad[src] = acc;
                }
    for (int64_t i = 0; i < g.P + bias; ++i) {
        const int64_t kh = i / (g.Kw * C), kw = (i % (g.Kw * C)) / C, c = i % C;
        for (int64_t kc = 0; kc < Kc; ++kc) {
            float acc = 0.0f;
            for (int64_t s = 0; s < g.S; ++s) {
                const int64_t a = s / (g.Nh * g.Nw), nh = (s % (g.Nh * g.Nw)) / g.Nw, nw = s % g.Nw;
                const int64_t k = s * Kc + kc;
                if (i == g.P) {
                    if (oldout[k] < max_cmp) {
                        prod = xbias - oldout[k]; prod = grad[k] * prod; prod = prod / wsum[k];
                        acc += prod;
                    }
                    continue;
                }
                const float v = xpad[((a * H + nh * g.Sh + kh) * W + nw * g.Sw + kw) * C + c];
                if (v >= max_cmp) continue;
                if (v < oldout[k] && oldout[k] < max_cmp) {
                    prod = v - oldout[k]; prod = grad[k] * prod; prod = prod / wsum[k];
                    acc += prod;
                }
            }
            dw[i * Kc + kc] = acc;
        }
    }
    free(wsum);
    return 0;
}
