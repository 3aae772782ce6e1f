/*
 * snntc.h -- C ABI of the MI355X (gfx950) implementation of the four SNN-TC custom ops.
 *
 * One entry point per reference op; each replaces the op's OpKernel::Compute (shape rules, error
 * checks) together with its GPU functor (device work).  Paths below are relative to the
 * reference checkout.
 *
 *   snntc_fc_forward   <- SnnFcOp::Compute      snntc/snnfc_kernels.cc:160-207
 *                         SnnFcFunctor<GPU>     snntc/snnfc_kernels.cu.cc:93-194
 *                         REGISTER_OP("SnnFc")  snntc/snnfc_ops.cc:6-27
 *   snntc_fc_backward  <- SnnFcGradOp::Compute  snntc/snnfcgrad_kernels.cc:93-131
 *                         SnnFcGradFunctor<GPU> snntc/snnfcgrad_kernels.cu.cc:137-225
 *                         REGISTER_OP("SnnFcGrad") snntc/snnfcgrad_ops.cc:6-20
 *   snntc_cv_forward   <- SnnCvOp::Compute      snntc/snncv_kernels.cc:191-242
 *                         SnnCvFunctor<GPU>     snntc/snncv_kernels.cu.cc:95-210
 *                         REGISTER_OP("SnnCv")  snntc/snncv_ops.cc:6-32
 *   snntc_cv_backward  <- SnnCvGradOp::Compute  snntc/snncvgrad_kernels.cc:131-183
 *                         SnnCvGradFunctor<GPU> snntc/snncvgrad_kernels.cu.cc:164-263
 *                         REGISTER_OP("SnnCvGrad") snntc/snncvgrad_ops.cc:6-20
 *
 * Conventions
 *  - All tensors are float32, row-major (images NHWC), and live in DEVICE memory, except
 *    `params`, which is a HOST pointer (the reference pins it with HostMemory("params"),
 *    snntc/snnfc_kernels.cc:224, snntc/snncv_kernels.cc:259).
 *  - The caller owns every buffer, including the scratch `workspace` (device memory, 256-byte
 *    aligned, at least snntc_*_workspace_bytes() long).  The library allocates nothing, keeps no
 *    state between calls and is re-entrant.
 *  - Work is enqueued on `stream` (a hipStream_t passed as void*; NULL = the default stream) and
 *    the call returns without synchronising.
 *  - Every function returns SNNTC_OK (0) or one of the codes below; snntc_last_error() returns a
 *    thread-local text for the last failure.  Invalid-argument codes mirror the reference's
 *    OP_REQUIRES(... InvalidArgument) conditions one to one.
 *
 * Params vectors (float32, exactly as the reference's Python layers build them)
 *  dense [6]  (SNN_TC_Modules.py:48-49):   {MAX_SPIKE_TIME, Epsilon, Spike_Threshold,
 *                                           Thread_per_Block, Blocks, biasvolt}
 *  conv  [12] (SNN_TC_Modules.py:121-123): {MAX_SPIKE_TIME, Thread_per_Block, Blocks, Epsilon,
 *                                           Spike_Threshold, cudaflag, Kh, Kw, Sh, Sw,
 *                                           padding==SAME, biasvolt}
 *  biasvolt > 1e-8 means the weight matrix carries one extra (last) bias row.  Epsilon,
 *  Thread_per_Block, Blocks and cudaflag are accepted and ignored (launch shapes are chosen for
 *  gfx950 by the library; the reference's GPU scan does not read Epsilon either).
 */
#ifndef SNNTC_H_
#define SNNTC_H_

#include <stddef.h>
#include <stdint.h>

#if defined(__GNUC__)
#define SNNTC_API __attribute__((visibility("default")))
#else
#define SNNTC_API
#endif

#ifdef __cplusplus
extern "C" {
#endif

enum {
    SNNTC_OK = 0,
    SNNTC_ERR_DIM_MISMATCH = 1,   /* weight rows vs input size (+bias); grad rows != 2*batch    */
    SNNTC_ERR_TOO_LARGE = 2,      /* a tensor (or the patch matrix) exceeds INT32_MAX elements  */
    SNNTC_ERR_BAD_ARGUMENT = 3,   /* null pointer, negative size, kernel larger than the image  */
    SNNTC_ERR_WORKSPACE = 4,      /* workspace missing, misaligned or too small                  */
    SNNTC_ERR_UNSUPPORTED = 5,    /* segment longer than the largest supported one (2^24 inputs) */
    SNNTC_ERR_HIP = 6             /* a HIP runtime call or kernel launch failed                  */
};

/* Library identification: "snntc-hip gfx950 <version>". */
SNNTC_API const char* snntc_version(void);
/* Text of the last error raised on the calling thread ("" if none). */
SNNTC_API const char* snntc_last_error(void);
/* Fixed text for a status code. */
SNNTC_API const char* snntc_status_string(int status);

/* ---------------------------------------------------------------------------------------------
 * One-time set-up of a device (no counterpart in the reference, whose kernels need none).  Raises the
 * dynamic-LDS limit of every kernel instantiation and looks up the device's copy of the library's
 * static scratch array.  device < 0 means the current device.  Optional: every entry point performs
 * the same set-up on its first call on a device -- but that first call must then not happen while a
 * stream is being captured into a HIP graph (hipFuncSetAttribute is not allowed there).  A caller
 * that captures graphs calls snntc_init() once per device beforehand, or runs one un-captured call.
 * ------------------------------------------------------------------------------------------- */
SNNTC_API int snntc_init(int device);

/* ---------------------------------------------------------------------------------------------
 * Dense layer (SNN_dense).   x[B,I]   w[w_rows,J] with w_rows == I + (biasvolt > 1e-8)
 * ------------------------------------------------------------------------------------------- */

/* Scratch sizes.  Replaces the reference's allocate_temp calls (snntc/snnfc_kernels.cu.cc:110-137,
 * snntc/snnfcgrad_kernels.cu.cc:159-164).  Inputs longer than 8192 per segment (I here, Kh*Kw*C
 * for conv layers) are sorted in pieces and merged in device memory; the forward size then includes
 * two key buffers for the merge passes.  Segments beyond 2^24 inputs -> UNSUPPORTED. */
SNNTC_API int snntc_fc_forward_workspace_bytes(int64_t B, int64_t I, int64_t J, size_t* bytes);
SNNTC_API int snntc_fc_backward_workspace_bytes(int64_t B, int64_t I, int64_t J, size_t* bytes);

/* out[2B,J]: rows [0,B) = output spike times y (MAX_SPIKE_TIME for a neuron that never fires),
 * rows [B,2B) = 1/(sum_{causal set} w - Spike_Threshold) (0 for a neuron that never fires).
 * Errors: w_rows not in {I, I+1} or inconsistent with biasvolt -> DIM_MISMATCH
 *         (snntc/snnfc_kernels.cc:171-172); B*I, w_rows*J or 2*B*J > INT32_MAX -> TOO_LARGE
 *         (snntc/snnfc_kernels.cc:194-203).
 * Layers with a handful of outputs (fewer work items than compute units) run a kernel whose
 * wavefronts hand each other running sums through LDS behind a bounded wait; should that wait ever
 * run out, the affected (sample, neuron) entries of both halves of `out` are NaN and the call still
 * returns SNNTC_OK (the library never synchronises with the device).  It has not been observed.
 * snntc_scan_status() below reports it without a pass over the outputs. */
SNNTC_API int snntc_fc_forward(const float* x, const float* w, const float* params_host, float* out,
                     int64_t B, int64_t I, int64_t J, int64_t w_rows,
                     void* workspace, size_t workspace_bytes, void* stream);

/* Same as snntc_fc_forward with optional side outputs (any may be NULL):
 *   sorted_z[B,I]  each input row sorted ascending (stable: equal values keep index order)
 *   perm[B,I]      int32 source column of every sorted element
 *   causal_k[B,J]  int32 number of sorted inputs in the causal set, -1 if the neuron never fired
 * These are the reference's temporaries d_in / order (snntc/snnfc_kernels.cu.cc:110-155) and the
 * loop counter k at exit of SnnFcCudaOutKernel (snntc/snnfc_kernels.cu.cc:43-62). */
SNNTC_API int snntc_fc_forward_ex(const float* x, const float* w, const float* params_host, float* out,
                        float* sorted_z, int32_t* perm, int32_t* causal_k,
                        int64_t B, int64_t I, int64_t J, int64_t w_rows,
                        void* workspace, size_t workspace_bytes, void* stream);

/* snntc_fc_forward for callers that cannot allocate device memory or carry a workspace: code under
 * HIP graph capture, tight serving loops, harnesses that forbid hipMalloc.  It has no counterpart
 * in the reference (whose ops allocate their temporaries through the framework on every call).
 * Same results as snntc_fc_forward, bit for bit; the scratch (sorted rows, permutation, counts)
 * lives in a static device array of SNNTC_STATIC_SCRATCH_BYTES inside the library, which every GPU
 * the library runs on holds until the process ends.  The call allocates and frees nothing.
 * Limits: snntc_fc_forward_workspace_bytes(B, I, J) must not exceed SNNTC_STATIC_SCRATCH_BYTES
 * (e.g. B = 1024 rows of I = 784), else SNNTC_ERR_WORKSPACE.  All calls on one GPU share that GPU's
 * array: calls that overlap in time on the same GPU (two streams, two threads) race; serialise them. */
#define SNNTC_STATIC_SCRATCH_BYTES (8u << 20)
SNNTC_API size_t snntc_static_scratch_bytes(void);
SNNTC_API int snntc_fc_forward_static(const float* x, const float* w, const float* params_host, float* out,
                            int64_t B, int64_t I, int64_t J, int64_t w_rows, void* stream);

/* grad[grad_rows,J] (only rows [0,B) are read, so a buffer holding just those rows may be passed with
 * grad_rows still declared as 2B), oldout[2B,J] = the forward output.
 * dx[B,I], dw[w_rows,J], dparams[6] (device; written with zeros).  Any of the three outputs may be
 * NULL: that gradient is then not computed (the reference always computes all of them).
 * Domain: inputs are spike times; dw is exact for x >= -MAX_SPIKE_TIME (it is formed from the
 * differences y - x, which the kernels keep within 2 * MAX_SPIKE_TIME; the same holds for
 * snntc_cv_backward).
 * Errors: grad_rows != 2B -> DIM_MISMATCH (snntc/snnfcgrad_kernels.cc:119-120); sizes as above. */
SNNTC_API int snntc_fc_backward(const float* grad, const float* x, const float* w, const float* params_host,
                      const float* oldout, float* dx, float* dw, float* dparams,
                      int64_t B, int64_t I, int64_t J, int64_t w_rows, int64_t grad_rows,
                      void* workspace, size_t workspace_bytes, void* stream);

/* ---------------------------------------------------------------------------------------------
 * Convolutional layer (SNN_conv).  xpad[B,H,W,C] is the input AFTER the Python layer's padding /
 * cropping (SNN_TC_Modules.py:144-166); w[w_rows,Kc] with w_rows == Kh*Kw*C + (biasvolt > 1e-8);
 * Nh = (H-Kh)/Sh + 1, Nw = (W-Kw)/Sw + 1 (snntc/snncv_kernels.cc:215).
 * ------------------------------------------------------------------------------------------- */

/* Output spatial size for a padded input, from the params vector. */
SNNTC_API int snntc_cv_output_dims(int64_t H, int64_t W, const float* params_host, int64_t* Nh, int64_t* Nw);

SNNTC_API int snntc_cv_forward_workspace_bytes(int64_t B, int64_t H, int64_t W, int64_t C, int64_t Kc,
                                     const float* params_host, size_t* bytes);
SNNTC_API int snntc_cv_backward_workspace_bytes(int64_t B, int64_t H, int64_t W, int64_t C, int64_t Kc,
                                      const float* params_host, size_t* bytes);

/* out[2B,Nh,Nw,Kc], halves as in the dense op.
 * Errors: w_rows != Kh*Kw*C + bias -> DIM_MISMATCH (snntc/snncv_kernels.cc:218); input, weight,
 *         output or B*Nh*Nw*w_rows > INT32_MAX -> TOO_LARGE (snntc/snncv_kernels.cc:231-238). */
SNNTC_API int snntc_cv_forward(const float* xpad, const float* w, const float* params_host, float* out,
                     int64_t B, int64_t H, int64_t W, int64_t C, int64_t Kc, int64_t w_rows,
                     void* workspace, size_t workspace_bytes, void* stream);

/* Side outputs per patch s=(b*Nh+nh)*Nw+nw, element order (kh,kw,c):
 *   sorted_z[B*Nh*Nw, Kh*Kw*C], perm[B*Nh*Nw, Kh*Kw*C], causal_k[B*Nh*Nw, Kc]. */
SNNTC_API int snntc_cv_forward_ex(const float* xpad, const float* w, const float* params_host, float* out,
                        float* sorted_z, int32_t* perm, int32_t* causal_k,
                        int64_t B, int64_t H, int64_t W, int64_t C, int64_t Kc, int64_t w_rows,
                        void* workspace, size_t workspace_bytes, void* stream);

/* snntc_cv_forward that also leaves the spike times where the next layer reads them: next_xpad is the
 * next SNN_conv's padded input, [B, next_h, next_w, Kc], and the time of output pixel (nh, nw) is
 * written to its pixel (nh + next_top, nw + next_left) as well as to `out`.  The border of next_xpad
 * (the layer's MAX_SPIKE_TIME padding, SNN_TC_Modules.py:147-161) is the caller's: it is constant, so it
 * is filled once when the buffer is made, not per call.  This replaces the tf.pad between two conv
 * layers of the reference's models (snntc/snntc-cifar10.py:73-106 stacks SNN_conv layers directly).
 * Errors: as snntc_cv_forward; an output that does not fit the destination at that offset -> BAD_ARGUMENT. */
SNNTC_API int snntc_cv_forward_chained(const float* xpad, const float* w, const float* params_host, float* out,
                             float* next_xpad, int64_t next_h, int64_t next_w, int64_t next_top, int64_t next_left,
                             int64_t B, int64_t H, int64_t W, int64_t C, int64_t Kc, int64_t w_rows,
                             void* workspace, size_t workspace_bytes, void* stream);

/* grad[grad_rows,Nh,Nw,Kc] (rows [0,B) read), oldout[2B,Nh,Nw,Kc].
 * dxpad[B,H,W,C] (gradient w.r.t. the padded input), dw[w_rows,Kc], dparams[12]; any may be NULL
 * (not computed).
 * Errors: grad_rows != 2B -> DIM_MISMATCH; sizes as in the forward op. */
SNNTC_API int snntc_cv_backward(const float* grad, const float* xpad, const float* w, const float* params_host,
                      const float* oldout, float* dxpad, float* dw, float* dparams,
                      int64_t B, int64_t H, int64_t W, int64_t C, int64_t Kc, int64_t w_rows,
                      int64_t grad_rows, void* workspace, size_t workspace_bytes, void* stream);

/* snntc_cv_backward that stores only a window of the padded input's gradient:
 *   dx[B, dx_h, dx_w, C] = dxpad[:, dx_top : dx_top + dx_h, dx_left : dx_left + dx_w, :].
 * With the window of the un-padded image this is the gradient the layer before expects, i.e. the
 * backward of the tf.pad in SNN_conv.__call__ (SNN_TC_Modules.py:147-161) folded into the op.
 * Errors: as snntc_cv_backward; a window that does not lie inside the padded image -> BAD_ARGUMENT. */
SNNTC_API int snntc_cv_backward_cropped(const float* grad, const float* xpad, const float* w, const float* params_host,
                              const float* oldout, float* dx, int64_t dx_h, int64_t dx_w, int64_t dx_top,
                              int64_t dx_left, float* dw, float* dparams, int64_t B, int64_t H, int64_t W, int64_t C,
                              int64_t Kc, int64_t w_rows, int64_t grad_rows, void* workspace, size_t workspace_bytes,
                              void* stream);

/* ---------------------------------------------------------------------------------------------
 * Loss of the example networks, loss_func (SNN_TC_Modules.py:286-288): categorical cross-entropy of
 * label[B,J] (one-hot, or any non-negative weights) against softmax(-times[B,J]).
 *   sample_loss[B]  per-sample loss  -sum_j label_j * log softmax(-times)_j        (may be NULL)
 *   dtimes[B,J]     gradient of the batch MEAN of sample_loss w.r.t. times         (may be NULL)
 * The batch mean itself is left to the caller (mean of sample_loss).  No workspace.
 * ------------------------------------------------------------------------------------------- */
SNNTC_API int snntc_softmax_time_loss(const float* times, const float* label, float* sample_loss, float* dtimes,
                            int64_t B, int64_t J, void* stream);

/* ---------------------------------------------------------------------------------------------
 * Earliest-spike pooling of NHWC spike times, SNN_maxpool2d (SNN_TC_Modules.py:215-246: pad with
 * padvalue = 1e5, then -maxpool(-x) with VALID windows).  The padding is implicit here:
 *   y[b,nh,nw,c] = min over kh < Kh, kw < Kw of x[b, nh*Sh - pad_top + kh, nw*Sw - pad_left + kw, c],
 * where positions outside the H x W image count as pad_value.  The caller passes the layer's
 * geometry: pad_top / pad_left (0 for VALID; the reference's SAME split puts int(total/2) before)
 * and Nh, Nw = the number of whole windows of the padded image.
 *   arg[b,nh,nw,c]  int32, kh*Kw + kw of the first window position (kh-major order) that attains
 *                   the minimum -- the position a max pooling of -x that replaces its running
 *                   maximum only on a strictly greater value ends on.  May be NULL (no backward).
 * Backward: dx[b,h,w,c] = sum of grad_y over the windows whose recorded position is pixel (h,w)
 * (a window whose minimum lies in the padding passes nothing on), added in (kh, kw) order.
 * No workspace.  Errors: a size < 0, Kh/Kw/Sh/Sw < 1, a pad < 0 or >= the kernel size, a window
 * that does not fit the padded image -> BAD_ARGUMENT; more than INT32_MAX elements -> TOO_LARGE.
 * ------------------------------------------------------------------------------------------- */
SNNTC_API int snntc_min_pool_forward(const float* x, float* y, int32_t* arg, int64_t B, int64_t H, int64_t W,
                           int64_t C, int64_t Kh, int64_t Kw, int64_t Sh, int64_t Sw, int64_t pad_top,
                           int64_t pad_left, int64_t Nh, int64_t Nw, float pad_value, void* stream);
/* snntc_min_pool_forward that also leaves the pooled times inside the padded input of the SNN_conv that
 * follows (next_xpad[B, next_h, next_w, C], pixel offset (next_top, next_left), border filled by the
 * caller): see snntc_cv_forward_chained. */
SNNTC_API int snntc_min_pool_forward_chained(const float* x, float* y, int32_t* arg, float* next_xpad, int64_t next_h,
                                   int64_t next_w, int64_t next_top, int64_t next_left, int64_t B, int64_t H, int64_t W,
                                   int64_t C, int64_t Kh, int64_t Kw, int64_t Sh, int64_t Sw, int64_t pad_top,
                                   int64_t pad_left, int64_t Nh, int64_t Nw, float pad_value, void* stream);
SNNTC_API int snntc_min_pool_backward(const float* grad_y, const int32_t* arg, float* dx, int64_t B, int64_t H,
                            int64_t W, int64_t C, int64_t Kh, int64_t Kw, int64_t Sh, int64_t Sw,
                            int64_t pad_top, int64_t pad_left, int64_t Nh, int64_t Nw, void* stream);

/* ---------------------------------------------------------------------------------------------
 * SAME padding of SNN_conv (SNN_TC_Modules.py:147-161: tf.pad with MAX_SPIKE_TIME) in one pass:
 *   xpad[b,hp,wp,c] = x[b, hp - top, wp - left, c] inside the H x W image, `value` outside,
 * xpad being [B,Hp,Wp,C] with Hp >= top + H, Wp >= left + W.  snntc_pad_time_backward is the
 * gradient: dx[b,h,w,c] = dxpad[b, h + top, w + left, c].  No workspace.
 * Errors: a negative size or offset, Hp < top + H, Wp < left + W -> BAD_ARGUMENT; more than
 * INT32_MAX elements -> TOO_LARGE.
 * ------------------------------------------------------------------------------------------- */
SNNTC_API int snntc_pad_time_forward(const float* x, float* xpad, int64_t B, int64_t H, int64_t W, int64_t C,
                           int64_t top, int64_t left, int64_t Hp, int64_t Wp, float value, void* stream);
SNNTC_API int snntc_pad_time_backward(const float* dxpad, float* dx, int64_t B, int64_t H, int64_t W, int64_t C,
                            int64_t top, int64_t left, int64_t Hp, int64_t Wp, void* stream);

/* ---------------------------------------------------------------------------------------------
 * SGD update of a training step: w[t][e] -= lr * dw[t][e] for e in [0, n[t]), t in [0, count).
 * The reference leaves the update to the framework's optimizer (snntc/snntc-mnist.py:70,92-93);
 * here all weight tensors of a network are updated by one launch (per 32 tensors).
 * w, dw and n are HOST arrays of `count` entries holding device pointers / element counts; they
 * are read before the call returns.  Tensors with n[t] == 0 are skipped.
 * Errors: count < 0, n[t] < 0, a NULL array or a NULL tensor with n[t] > 0 -> BAD_ARGUMENT.
 * ------------------------------------------------------------------------------------------- */
SNNTC_API int snntc_sgd_update(float* const* w, const float* const* dw, const int64_t* n, int64_t count, float lr,
                     void* stream);

/* ---------------------------------------------------------------------------------------------
 * Health of the bounded wait described at snntc_fc_forward (no counterpart in the reference, whose scan
 * has one thread per neuron and nothing to wait for).
 *   snntc_scan_status(&giveups, stream)  number of wavefronts, on the current device since the process
 *       started, whose wait ran out (each poisons the outputs of its work item with NaN).  0 = every scan
 *       result so far is what the kernels computed.  The count is a 4-byte device word read with a copy on
 *       `stream` followed by a wait for that stream: call it where the caller synchronises anyway (after a
 *       training step's loss has been read, at the end of a batch of requests).
 *   snntc_debug_set_scan_wait_polls(polls)  test hook: the number of polls a waiting wavefront spends from
 *       the next launch on (process-wide; polls < 0 restores the default of 2^20).  With 0 every wait that
 *       is not already satisfied at its first poll gives up, which drives the give-up path while every
 *       kernel still runs to its end.
 * ------------------------------------------------------------------------------------------- */
SNNTC_API int snntc_scan_status(int64_t* giveups, void* stream);
SNNTC_API int snntc_debug_set_scan_wait_polls(int polls);

/* ---------------------------------------------------------------------------------------------
 * Per-kernel timing (no counterpart in the reference, which only times whole scripts with
 * time.time()).  While enabled, every kernel the library launches is bracketed by a pair of HIP
 * events on its launch stream; this is the only process-wide state the library keeps and it is
 * off by default.
 *   snntc_profile_enable(1|0)  clear the totals and switch timing on / off
 *   snntc_profile_collect()    wait for the recorded events, fold them into per-kernel totals and
 *                              return the number of distinct kernels seen (>= 0)
 *   snntc_profile_entry(i,...) name, launch count and summed duration (ms) of kernel i; `name`
 *                              stays valid until the next collect/enable call
 * ------------------------------------------------------------------------------------------- */
SNNTC_API int snntc_profile_enable(int on);
SNNTC_API int snntc_profile_collect(void);
SNNTC_API int snntc_profile_entry(int index, const char** name, int64_t* launches, double* total_ms);

#ifdef __cplusplus
}
#endif
#endif /* SNNTC_H_ */
