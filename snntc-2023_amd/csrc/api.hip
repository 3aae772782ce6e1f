// C ABI of the library (declared in include/snntc.h): argument checks that mirror the reference
// OpKernels' OP_REQUIRES conditions, workspace carving, and the kernel chains of the four ops.
#include <limits.h>
#include <stdarg.h>
#include <stdio.h>
#include <string.h>

#include <map>
#include <mutex>
#include <string>
#include <vector>

#include "snntc_common.h"

// Library-owned scratch of snntc_fc_forward_static (the entry point that allocates nothing): held by
// every GPU the library runs on until the process ends.  Host code never passes this name to a
// kernel; it asks hipGetSymbolAddress for the device's copy once (prepare_device below).
static __device__ __align__(256) unsigned char scratch[SNNTC_STATIC_SCRATCH_BYTES];

namespace snntc {

static thread_local char g_last_error[512] = "";

// ---- opt-in kernel timer ---------------------------------------------------------------------
namespace {
struct TimedLaunch { const char* name; hipEvent_t start, stop; };
struct TimerTotals { int64_t launches = 0; double ms = 0.0; };
std::mutex g_prof_mutex;
bool g_prof_enabled = false;
std::vector<TimedLaunch> g_prof_pending;
std::map<std::string, TimerTotals> g_prof_totals;
std::vector<std::pair<std::string, TimerTotals>> g_prof_snapshot;

// Waits for every pending event pair and folds it into the totals.  Caller holds the mutex.
void prof_drain() {
    for (TimedLaunch& t : g_prof_pending) {
        float ms = 0.0f;
        if (hipEventSynchronize(t.stop) == hipSuccess && hipEventElapsedTime(&ms, t.start, t.stop) == hipSuccess) {
            TimerTotals& tot = g_prof_totals[t.name];
            tot.launches += 1;
            tot.ms += ms;
        }
        (void)hipEventDestroy(t.start);
        (void)hipEventDestroy(t.stop);
    }
    g_prof_pending.clear();
}
}  // namespace

KernelTimerScope::KernelTimerScope(const char* name, hipStream_t st) : slot(-1), stream(st) {
    if (!g_prof_enabled) return;
    std::lock_guard<std::mutex> lock(g_prof_mutex);
    TimedLaunch t{name, nullptr, nullptr};
    if (hipEventCreate(&t.start) != hipSuccess) return;
    if (hipEventCreate(&t.stop) != hipSuccess) { (void)hipEventDestroy(t.start); return; }
    (void)hipEventRecord(t.start, stream);
    g_prof_pending.push_back(t);
    slot = (int)g_prof_pending.size() - 1;
}

KernelTimerScope::~KernelTimerScope() {
    if (slot < 0) return;
    std::lock_guard<std::mutex> lock(g_prof_mutex);
    if (slot < (int)g_prof_pending.size()) (void)hipEventRecord(g_prof_pending[slot].stop, stream);
}

int fail(int code, const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_last_error, sizeof(g_last_error), fmt, ap);
    va_end(ap);
    return code;
}

namespace {

constexpr int64_t kInt32Max = INT32_MAX;

NeuronParams neuron_params(float max_time, float theta, float biasvolt) {
    NeuronParams np;
    np.max_time = max_time;
    np.max_cmp = max_time - 0.1f;
    np.theta = theta;
    np.biasvolt = biasvolt;
    np.bias = biasvolt > 1e-8f ? 1 : 0;
    np.wait_polls = 0;                                    // the scan launcher fills it in
    return np;
}

// Hands out 256-byte aligned pieces of the caller's workspace.
struct Carver {
    char* base;
    size_t used = 0;
    explicit Carver(void* p) : base(static_cast<char*>(p)) {}
    template <typename T>
    T* take(int64_t count) {
        T* p = base ? reinterpret_cast<T*>(base + used) : nullptr;
        used += align_up((size_t)(count > 0 ? count : 0) * sizeof(T));
        return p;
    }
};

int check_workspace(const void* ws, size_t have, size_t need) {
    if (need == 0) return SNNTC_OK;
    if (!ws) return fail(SNNTC_ERR_WORKSPACE, "workspace is NULL but %zu bytes are required", need);
    if (reinterpret_cast<uintptr_t>(ws) % kAlign != 0)
        return fail(SNNTC_ERR_WORKSPACE, "workspace must be %zu-byte aligned", kAlign);
    if (have < need) return fail(SNNTC_ERR_WORKSPACE, "workspace too small: %zu bytes given, %zu required", have, need);
    return SNNTC_OK;
}

// ---- dense -------------------------------------------------------------------------------------

int fc_check(int64_t B, int64_t I, int64_t J, int64_t w_rows, const float* params, const char* who) {
    if (!params) return fail(SNNTC_ERR_BAD_ARGUMENT, "%s: params is NULL", who);
    if (B < 0 || I < 1 || J < 0) return fail(SNNTC_ERR_BAD_ARGUMENT, "%s: bad sizes B=%lld I=%lld J=%lld", who,
                                              (long long)B, (long long)I, (long long)J);
    const int bias = params[5] > 1e-8f ? 1 : 0;
    if (w_rows != I && w_rows != I + 1)
        return fail(SNNTC_ERR_DIM_MISMATCH, "%s: Input & Weight inner-dim mismatch (input %lld, weight rows %lld)",
                    who, (long long)I, (long long)w_rows);
    if (w_rows != I + bias)
        return fail(SNNTC_ERR_DIM_MISMATCH, "%s: weight rows %lld do not match input %lld with biasvolt %g", who,
                    (long long)w_rows, (long long)I, (double)params[5]);
    if (B * I > kInt32Max) return fail(SNNTC_ERR_TOO_LARGE, "%s: Too many elements in input tensor", who);
    if (w_rows * J > kInt32Max) return fail(SNNTC_ERR_TOO_LARGE, "%s: Too many elements in weight tensor", who);
    if (2 * B * J > kInt32Max) return fail(SNNTC_ERR_TOO_LARGE, "%s: Too many elements in output tensor", who);
    if (I > kMaxLongSegment)
        return fail(SNNTC_ERR_UNSUPPORTED, "%s: input size %lld exceeds the largest supported segment (%d)", who,
                    (long long)I, kMaxLongSegment);
    return SNNTC_OK;
}

// Forward scratch.  n_pix / pix_c > 0 adds the per-pixel sorted channels the conv merge path needs.
struct FcFwdWs {
    float* sorted; int32_t* perm; int32_t* n_real; float* pix_z; int32_t* pix_c;
    void* long_keys;                                      // merge passes of segments longer than one network
    int64_t stride, pix_stride; size_t bytes;
};
FcFwdWs fc_fwd_ws(void* ws, int64_t S, int64_t I, int64_t n_pix = 0, int64_t pix_c = 0) {
    Carver c(ws);
    FcFwdWs r;
    r.stride = padded_stride(I);
    r.pix_stride = padded_stride(pix_c);
    r.sorted = c.take<float>(S * r.stride);
    r.perm = c.take<int32_t>(S * r.stride);
    r.n_real = c.take<int32_t>(S);
    r.pix_z = c.take<float>(n_pix * r.pix_stride);
    r.pix_c = c.take<int32_t>(n_pix * r.pix_stride);
    const size_t long_bytes = sort_long_workspace_bytes(S, I);
    r.long_keys = long_bytes ? c.take<unsigned char>((int64_t)long_bytes) : nullptr;
    r.bytes = c.used;
    return r;
}

// sort -> (optional copy of the side outputs) -> scan, shared by the dense and the conv op
int forward_chain(const SegmentSource& src, const FcFwdWs& ws, const float* w, float* out, float* sorted_z,
                  int32_t* perm, int32_t* causal_k, int64_t S, int64_t I, int64_t J, const NeuronParams& np,
                  const TimeCopy& copy, hipStream_t st) {
    int rc = launch_sort(src, S, ws.sorted, ws.perm, ws.n_real, (int)ws.stride, np.max_cmp, ws.long_keys, st);
    if (rc) return rc;
    rc = launch_unpad_rows(ws.sorted, ws.perm, sorted_z, perm, S, I, ws.stride, st);
    if (rc) return rc;
    return launch_scan(ws.sorted, ws.perm, ws.n_real, w, out, out + S * J, causal_k, S, I, ws.stride, J, np, copy, st);
}

// Backward scratch.  `rows` is the weight row count including a possible bias row; the partial-sum
// area is sized for the worst case of 256 slices only when slicing can happen at all.
struct BwdWs { float* upm; float* wt; float* dxp; float* partial; int max_split; size_t bytes; };
// patch_scratch: elements of the per-patch gradient of conv layers whose dX goes through patch space
// narrow_split: slices the one-launch backward of a narrow dense layer needs (0: not that path)
BwdWs bwd_ws(void* ws, int64_t S, int64_t rows, int64_t J, int64_t min_base_blocks, int64_t patch_scratch = 0,
             int narrow_split = 0) {
    Carver c(ws);
    BwdWs r;
    r.upm = c.take<float>(S * J);
    r.wt = c.take<float>(rows * J);
    r.dxp = c.take<float>(patch_scratch);
    r.max_split = weight_grad_splits(S, min_base_blocks);
    if (narrow_split > r.max_split) r.max_split = narrow_split;
    r.partial = c.take<float>(r.max_split > 1 ? (int64_t)r.max_split * rows * J : 0);
    r.bytes = c.used;
    return r;
}

// Smallest block count the weight-gradient launch of a conv layer can have (it decides how far the
// patch range may be sliced): the wide kernel covers 32 rows per block, the generic one 8.
int64_t cv_weight_base_blocks(const ConvGeom& g) {
    const int64_t generic = grad_weight_blocks(g.P + 1, g.Kc);
    const int64_t wide = cv_grad_weight_wide_supported(g) ? cv_grad_weight_wide_blocks(g) : generic;
    return wide < generic ? wide : generic;
}

int fc_forward_impl(const float* x, const float* w, const float* params, float* out, float* sorted_z,
                    int32_t* perm, int32_t* causal_k, int64_t B, int64_t I, int64_t J, int64_t w_rows,
                    void* workspace, size_t workspace_bytes, void* stream) {
    int rc = fc_check(B, I, J, w_rows, params, "snntc_fc_forward");
    if (rc) return rc;
    if (B == 0 || J == 0) return SNNTC_OK;
    if (!x || !w || !out) return fail(SNNTC_ERR_BAD_ARGUMENT, "snntc_fc_forward: NULL tensor pointer");
    FcFwdWs ws = fc_fwd_ws(workspace, B, I);
    rc = check_workspace(workspace, workspace_bytes, ws.bytes);
    if (rc) return rc;
    hipStream_t st = static_cast<hipStream_t>(stream);
    const NeuronParams np = neuron_params(params[0], params[2], params[5]);
    SegmentSource src{};
    src.base = x; src.conv = 0; src.I = (int)I;
    return forward_chain(src, ws, w, out, sorted_z, perm, causal_k, B, I, J, np, TimeCopy{}, st);
}

// ---- conv --------------------------------------------------------------------------------------

int cv_geom(int64_t B, int64_t H, int64_t W, int64_t C, int64_t Kc, int64_t w_rows, const float* params,
            bool check_rows, const char* who, ConvGeom* g) {
    if (!params) return fail(SNNTC_ERR_BAD_ARGUMENT, "%s: params is NULL", who);
    g->B = B; g->H = H; g->W = W; g->C = C; g->Kc = Kc;
    g->Kh = (int64_t)params[6]; g->Kw = (int64_t)params[7];
    g->Sh = (int64_t)params[8]; g->Sw = (int64_t)params[9];
    if (B < 0 || H < 1 || W < 1 || C < 1 || Kc < 0)
        return fail(SNNTC_ERR_BAD_ARGUMENT, "%s: bad sizes B=%lld H=%lld W=%lld C=%lld Kc=%lld", who, (long long)B,
                    (long long)H, (long long)W, (long long)C, (long long)Kc);
    if (g->Kh < 1 || g->Kw < 1 || g->Sh < 1 || g->Sw < 1)
        return fail(SNNTC_ERR_BAD_ARGUMENT, "%s: bad kernel/stride in params (Kh=%lld Kw=%lld Sh=%lld Sw=%lld)", who,
                    (long long)g->Kh, (long long)g->Kw, (long long)g->Sh, (long long)g->Sw);
    if (g->Kh > H || g->Kw > W)
        return fail(SNNTC_ERR_BAD_ARGUMENT, "%s: kernel %lldx%lld larger than the (padded) input %lldx%lld", who,
                    (long long)g->Kh, (long long)g->Kw, (long long)H, (long long)W);
    g->Nh = (H - g->Kh) / g->Sh + 1;
    g->Nw = (W - g->Kw) / g->Sw + 1;
    g->P = g->Kh * g->Kw * C;
    g->S = B * g->Nh * g->Nw;
    if (!check_rows) return SNNTC_OK;
    const int bias = params[11] > 1e-8f ? 1 : 0;
    if (w_rows != g->P + bias)
        return fail(SNNTC_ERR_DIM_MISMATCH, "%s: Input & Weight dim mismatch (bias): weight rows %lld, expected %lld",
                    who, (long long)w_rows, (long long)(g->P + bias));
    if (B * H * W * C > kInt32Max) return fail(SNNTC_ERR_TOO_LARGE, "%s: Too many elements in input tensor", who);
    if (w_rows * Kc > kInt32Max) return fail(SNNTC_ERR_TOO_LARGE, "%s: Too many elements in weight tensor", who);
    if (2 * g->S * Kc > kInt32Max) return fail(SNNTC_ERR_TOO_LARGE, "%s: Too many elements in output tensor", who);
    if (g->S * w_rows > kInt32Max) return fail(SNNTC_ERR_TOO_LARGE, "%s: Too many elements in patched tensor", who);
    if (g->P > kMaxLongSegment)
        return fail(SNNTC_ERR_UNSUPPORTED, "%s: patch length %lld exceeds the largest supported segment (%d)", who,
                    (long long)g->P, kMaxLongSegment);
    return SNNTC_OK;
}

SegmentSource conv_source(const float* xpad, const ConvGeom& g) {
    SegmentSource src{};
    src.base = xpad; src.conv = 1; src.I = (int)g.P;
    src.H = (int)g.H; src.W = (int)g.W; src.C = (int)g.C;
    src.Kh = (int)g.Kh; src.Kw = (int)g.Kw; src.Sh = (int)g.Sh; src.Sw = (int)g.Sw;
    src.Nh = (int)g.Nh; src.Nw = (int)g.Nw;
    return src;
}

// next_xpad (may be NULL): a second copy of the spike times, placed as pixel (nh + next_top, nw + next_left)
// of an image tensor [B, next_h, next_w, Kc]
int cv_forward_impl(const float* xpad, const float* w, const float* params, float* out, float* sorted_z,
                    int32_t* perm, int32_t* causal_k, float* next_xpad, int64_t next_h, int64_t next_w,
                    int64_t next_top, int64_t next_left, int64_t B, int64_t H, int64_t W, int64_t C, int64_t Kc,
                    int64_t w_rows, void* workspace, size_t workspace_bytes, void* stream) {
    ConvGeom g;
    int rc = cv_geom(B, H, W, C, Kc, w_rows, params, true, "snntc_cv_forward", &g);
    if (rc) return rc;
    TimeCopy copy{};
    if (next_xpad) {
        if (next_top < 0 || next_left < 0 || next_h < next_top + g.Nh || next_w < next_left + g.Nw)
            return fail(SNNTC_ERR_BAD_ARGUMENT, "snntc_cv_forward_chained: the %lld x %lld output does not fit the "
                        "%lld x %lld destination at offset (%lld, %lld)", (long long)g.Nh, (long long)g.Nw,
                        (long long)next_h, (long long)next_w, (long long)next_top, (long long)next_left);
        if (B * next_h * next_w * Kc > kInt32Max)
            return fail(SNNTC_ERR_TOO_LARGE, "snntc_cv_forward_chained: Too many elements in the destination tensor");
        copy = TimeCopy{next_xpad, (int)g.Nh, (int)g.Nw, (int)next_h, (int)next_w, (int)next_top, (int)next_left};
    }
    if (g.S == 0 || Kc == 0) return SNNTC_OK;
    if (!xpad || !w || !out) return fail(SNNTC_ERR_BAD_ARGUMENT, "snntc_cv_forward: NULL tensor pointer");
    const bool merge = merge_sort_supported(g);
    FcFwdWs ws = fc_fwd_ws(workspace, g.S, g.P, merge ? B * H * W : 0, merge ? C : 0);
    rc = check_workspace(workspace, workspace_bytes, ws.bytes);
    if (rc) return rc;
    hipStream_t st = static_cast<hipStream_t>(stream);
    const NeuronParams np = neuron_params(params[0], params[4], params[11]);
    if (!merge)
        return forward_chain(conv_source(xpad, g), ws, w, out, sorted_z, perm, causal_k, g.S, g.P, Kc, np, copy, st);
    // sort every pixel's channels once, then assemble the patches by rank merging
    SegmentSource pixels{};
    pixels.base = xpad; pixels.conv = 0; pixels.I = (int)C;
    rc = launch_sort(pixels, B * H * W, ws.pix_z, ws.pix_c, nullptr, (int)ws.pix_stride, np.max_cmp, nullptr, st);
    if (rc) return rc;
    rc = launch_merge_patches(ws.pix_z, ws.pix_c, ws.pix_stride, ws.sorted, ws.perm, ws.n_real, g, ws.stride,
                              np.max_cmp, st);
    if (rc) return rc;
    rc = launch_unpad_rows(ws.sorted, ws.perm, sorted_z, perm, g.S, g.P, ws.stride, st);
    if (rc) return rc;
    return launch_scan(ws.sorted, ws.perm, ws.n_real, w, out, out + g.S * Kc, causal_k, g.S, g.P, ws.stride, Kc, np,
                       copy, st);
}


// ---- per-device one-time set-up and the library-owned scratch of snntc_fc_forward_static ----------
// `scratch` is the forward workspace of the allocation-free entry point.  In host code the array's
// name is only a handle for hipGetSymbolAddress: the device address (each GPU holds its own copy)
// is looked up once per device and kept in g_scratch_ptr; host code uses that pointer, never the name.
constexpr size_t kStaticScratchBytes = SNNTC_STATIC_SCRATCH_BYTES;

std::mutex g_init_mutex;
void* g_scratch_ptr[kMaxDevices];          // device address of `scratch` on each device, NULL until set up

// Set-up of the current device `dev`: dynamic-LDS limits of all kernels and the address of `scratch`.
int prepare_device(int dev, void** scratch_out) {
    if (dev < 0 || dev >= kMaxDevices)
        return fail(SNNTC_ERR_UNSUPPORTED, "snntc_init: device index %d not supported", dev);
    std::lock_guard<std::mutex> lock(g_init_mutex);
    if (!g_scratch_ptr[dev]) {
        int rc = scan_prepare_device(dev, nullptr);
        if (!rc) rc = merge_prepare_device(dev);
        if (rc) return rc;
        void* ptr = nullptr;
        SNNTC_HIP_CHECK(hipGetSymbolAddress(&ptr, HIP_SYMBOL(::scratch)));
        if (!ptr || reinterpret_cast<uintptr_t>(ptr) % kAlign != 0)
            return fail(SNNTC_ERR_HIP, "snntc_init: the static scratch array has no usable device address");
        g_scratch_ptr[dev] = ptr;
    }
    if (scratch_out) *scratch_out = g_scratch_ptr[dev];
    return SNNTC_OK;
}

}  // namespace
}  // namespace snntc

using namespace snntc;

extern "C" {

const char* snntc_version(void) { return "snntc-hip gfx950 0.1"; }

const char* snntc_last_error(void) { return g_last_error; }

const char* snntc_status_string(int status) {
    switch (status) {
        case SNNTC_OK: return "ok";
        case SNNTC_ERR_DIM_MISMATCH: return "tensor dimension mismatch";
        case SNNTC_ERR_TOO_LARGE: return "tensor exceeds INT32_MAX elements";
        case SNNTC_ERR_BAD_ARGUMENT: return "bad argument";
        case SNNTC_ERR_WORKSPACE: return "workspace missing, misaligned or too small";
        case SNNTC_ERR_UNSUPPORTED: return "segment longer than the largest supported sort";
        case SNNTC_ERR_HIP: return "HIP runtime error";
        default: return "unknown status";
    }
}

int snntc_softmax_time_loss(const float* times, const float* label, float* sample_loss, float* dtimes, int64_t B,
                            int64_t J, void* stream) {
    if (B < 0 || J < 0) return fail(SNNTC_ERR_BAD_ARGUMENT, "snntc_softmax_time_loss: negative size");
    if (B > INT32_MAX || J > INT32_MAX || B * J > INT32_MAX)
        return fail(SNNTC_ERR_TOO_LARGE, "snntc_softmax_time_loss: more than INT32_MAX elements");
    if (B > 0 && J > 0 && (!times || !label || (!sample_loss && !dtimes)))
        return fail(SNNTC_ERR_BAD_ARGUMENT, "snntc_softmax_time_loss: null pointer");
    return launch_softmax_time_loss(times, label, sample_loss, dtimes, B, J, static_cast<hipStream_t>(stream));
}

// Geometry checks shared by the two pooling entry points.
static int pool_geom(int64_t B, int64_t H, int64_t W, int64_t C, int64_t Kh, int64_t Kw, int64_t Sh, int64_t Sw,
                     int64_t pad_top, int64_t pad_left, int64_t Nh, int64_t Nw, const char* who, PoolGeom* g) {
    if (B < 0 || H < 0 || W < 0 || C < 0 || Nh < 0 || Nw < 0)
        return fail(SNNTC_ERR_BAD_ARGUMENT, "%s: negative size", who);
    if (Kh < 1 || Kw < 1 || Sh < 1 || Sw < 1) return fail(SNNTC_ERR_BAD_ARGUMENT, "%s: kernel and stride must be >= 1", who);
    if (pad_top < 0 || pad_left < 0 || pad_top >= Kh || pad_left >= Kw)
        return fail(SNNTC_ERR_BAD_ARGUMENT, "%s: padding %lld x %lld outside [0, kernel)", who, (long long)pad_top,
                    (long long)pad_left);
    // every window has to reach into the image (a window wholly inside the padding has no meaning)
    if (Nh > 0 && (Nh - 1) * Sh - pad_top >= H) return fail(SNNTC_ERR_BAD_ARGUMENT, "%s: Nh %lld does not fit", who, (long long)Nh);
    if (Nw > 0 && (Nw - 1) * Sw - pad_left >= W) return fail(SNNTC_ERR_BAD_ARGUMENT, "%s: Nw %lld does not fit", who, (long long)Nw);
    if (B * H * W * C > kInt32Max || B * Nh * Nw * C > kInt32Max)
        return fail(SNNTC_ERR_TOO_LARGE, "%s: more than INT32_MAX elements", who);
    *g = PoolGeom{B, H, W, C, Kh, Kw, Sh, Sw, pad_top, pad_left, Nh, Nw};
    return SNNTC_OK;
}

int snntc_min_pool_forward(const float* x, float* y, int32_t* arg, int64_t B, int64_t H, int64_t W, int64_t C,
                           int64_t Kh, int64_t Kw, int64_t Sh, int64_t Sw, int64_t pad_top, int64_t pad_left,
                           int64_t Nh, int64_t Nw, float pad_value, void* stream) {
    PoolGeom g;
    int rc = pool_geom(B, H, W, C, Kh, Kw, Sh, Sw, pad_top, pad_left, Nh, Nw, "snntc_min_pool_forward", &g);
    if (rc) return rc;
    if (B * Nh * Nw * C == 0) return SNNTC_OK;
    if (!y || (!x && B * H * W * C > 0)) return fail(SNNTC_ERR_BAD_ARGUMENT, "snntc_min_pool_forward: NULL tensor pointer");
    return launch_min_pool_forward(x, y, arg, g, pad_value, TimeCopy{}, static_cast<hipStream_t>(stream));
}

int snntc_min_pool_forward_chained(const float* x, float* y, int32_t* arg, float* next_xpad, int64_t next_h,
                                   int64_t next_w, int64_t next_top, int64_t next_left, int64_t B, int64_t H, int64_t W,
                                   int64_t C, int64_t Kh, int64_t Kw, int64_t Sh, int64_t Sw, int64_t pad_top,
                                   int64_t pad_left, int64_t Nh, int64_t Nw, float pad_value, void* stream) {
    PoolGeom g;
    int rc = pool_geom(B, H, W, C, Kh, Kw, Sh, Sw, pad_top, pad_left, Nh, Nw, "snntc_min_pool_forward_chained", &g);
    if (rc) return rc;
    if (!next_xpad) return fail(SNNTC_ERR_BAD_ARGUMENT, "snntc_min_pool_forward_chained: next_xpad is NULL");
    if (next_top < 0 || next_left < 0 || next_h < next_top + Nh || next_w < next_left + Nw)
        return fail(SNNTC_ERR_BAD_ARGUMENT, "snntc_min_pool_forward_chained: the %lld x %lld output does not fit the "
                    "%lld x %lld destination at offset (%lld, %lld)", (long long)Nh, (long long)Nw, (long long)next_h,
                    (long long)next_w, (long long)next_top, (long long)next_left);
    if (B * next_h * next_w * C > kInt32Max)
        return fail(SNNTC_ERR_TOO_LARGE, "snntc_min_pool_forward_chained: Too many elements in the destination tensor");
    if (B * Nh * Nw * C == 0) return SNNTC_OK;
    if (!y || (!x && B * H * W * C > 0))
        return fail(SNNTC_ERR_BAD_ARGUMENT, "snntc_min_pool_forward_chained: NULL tensor pointer");
    const TimeCopy copy{next_xpad, (int)Nh, (int)Nw, (int)next_h, (int)next_w, (int)next_top, (int)next_left};
    return launch_min_pool_forward(x, y, arg, g, pad_value, copy, static_cast<hipStream_t>(stream));
}

int snntc_min_pool_backward(const float* grad_y, const int32_t* arg, float* dx, int64_t B, int64_t H, int64_t W,
                            int64_t C, int64_t Kh, int64_t Kw, int64_t Sh, int64_t Sw, int64_t pad_top,
                            int64_t pad_left, int64_t Nh, int64_t Nw, void* stream) {
    PoolGeom g;
    int rc = pool_geom(B, H, W, C, Kh, Kw, Sh, Sw, pad_top, pad_left, Nh, Nw, "snntc_min_pool_backward", &g);
    if (rc) return rc;
    if (B * H * W * C == 0) return SNNTC_OK;
    if (!dx || ((!grad_y || !arg) && B * Nh * Nw * C > 0))
        return fail(SNNTC_ERR_BAD_ARGUMENT, "snntc_min_pool_backward: NULL tensor pointer");
    return launch_min_pool_backward(grad_y, arg, dx, g, static_cast<hipStream_t>(stream));
}

static int pad_geom(int64_t B, int64_t H, int64_t W, int64_t C, int64_t top, int64_t left, int64_t Hp, int64_t Wp,
                    const char* who, PadGeom* g) {
    if (B < 0 || H < 0 || W < 0 || C < 0 || top < 0 || left < 0)
        return fail(SNNTC_ERR_BAD_ARGUMENT, "%s: negative size or offset", who);
    if (Hp < top + H || Wp < left + W)
        return fail(SNNTC_ERR_BAD_ARGUMENT, "%s: padded size %lld x %lld does not hold the image", who, (long long)Hp,
                    (long long)Wp);
    if (B * Hp * Wp * C > kInt32Max) return fail(SNNTC_ERR_TOO_LARGE, "%s: more than INT32_MAX elements", who);
    *g = PadGeom{B, H, W, C, top, left, Hp, Wp};
    return SNNTC_OK;
}

int snntc_pad_time_forward(const float* x, float* xpad, int64_t B, int64_t H, int64_t W, int64_t C, int64_t top,
                           int64_t left, int64_t Hp, int64_t Wp, float value, void* stream) {
    PadGeom g;
    int rc = pad_geom(B, H, W, C, top, left, Hp, Wp, "snntc_pad_time_forward", &g);
    if (rc) return rc;
    if (B * Hp * Wp * C == 0) return SNNTC_OK;
    if (!xpad || (!x && B * H * W * C > 0)) return fail(SNNTC_ERR_BAD_ARGUMENT, "snntc_pad_time_forward: NULL tensor pointer");
    return launch_pad_time(x, xpad, g, value, static_cast<hipStream_t>(stream));
}

int snntc_pad_time_backward(const float* dxpad, float* dx, int64_t B, int64_t H, int64_t W, int64_t C, int64_t top,
                            int64_t left, int64_t Hp, int64_t Wp, void* stream) {
    PadGeom g;
    int rc = pad_geom(B, H, W, C, top, left, Hp, Wp, "snntc_pad_time_backward", &g);
    if (rc) return rc;
    if (B * H * W * C == 0) return SNNTC_OK;
    if (!dxpad || !dx) return fail(SNNTC_ERR_BAD_ARGUMENT, "snntc_pad_time_backward: NULL tensor pointer");
    return launch_crop_time(dxpad, dx, g, static_cast<hipStream_t>(stream));
}

int snntc_sgd_update(float* const* w, const float* const* dw, const int64_t* n, int64_t count, float lr,
                     void* stream) {
    if (count < 0 || count > INT32_MAX) return fail(SNNTC_ERR_BAD_ARGUMENT, "snntc_sgd_update: bad tensor count");
    if (count == 0) return SNNTC_OK;
    if (!w || !dw || !n) return fail(SNNTC_ERR_BAD_ARGUMENT, "snntc_sgd_update: null array");
    for (int64_t t = 0; t < count; ++t) {
        if (n[t] < 0) return fail(SNNTC_ERR_BAD_ARGUMENT, "snntc_sgd_update: tensor %lld has a negative size", (long long)t);
        if (n[t] > 0 && (!w[t] || !dw[t]))
            return fail(SNNTC_ERR_BAD_ARGUMENT, "snntc_sgd_update: tensor %lld is a null pointer", (long long)t);
    }
    return launch_sgd_update(w, dw, n, (int)count, lr, static_cast<hipStream_t>(stream));
}

int snntc_scan_status(int64_t* giveups, void* stream) {
    if (!giveups) return fail(SNNTC_ERR_BAD_ARGUMENT, "snntc_scan_status: giveups is NULL");
    return read_scan_giveups(giveups, static_cast<hipStream_t>(stream));
}

int snntc_debug_set_scan_wait_polls(int polls) {
    set_scan_wait_polls(polls);
    return SNNTC_OK;
}

int snntc_profile_enable(int on) {
    std::lock_guard<std::mutex> lock(g_prof_mutex);
    prof_drain();
    g_prof_totals.clear();
    g_prof_snapshot.clear();
    g_prof_enabled = on != 0;
    return SNNTC_OK;
}

int snntc_profile_collect(void) {
    std::lock_guard<std::mutex> lock(g_prof_mutex);
    prof_drain();
    g_prof_snapshot.assign(g_prof_totals.begin(), g_prof_totals.end());
    return (int)g_prof_snapshot.size();
}

int snntc_profile_entry(int index, const char** name, int64_t* launches, double* total_ms) {
    std::lock_guard<std::mutex> lock(g_prof_mutex);
    if (index < 0 || index >= (int)g_prof_snapshot.size())
        return fail(SNNTC_ERR_BAD_ARGUMENT, "snntc_profile_entry: index %d out of range", index);
    if (name) *name = g_prof_snapshot[index].first.c_str();
    if (launches) *launches = g_prof_snapshot[index].second.launches;
    if (total_ms) *total_ms = g_prof_snapshot[index].second.ms;
    return SNNTC_OK;
}

int snntc_fc_forward_workspace_bytes(int64_t B, int64_t I, int64_t J, size_t* bytes) {
    (void)J;
    if (!bytes || B < 0 || I < 0) return fail(SNNTC_ERR_BAD_ARGUMENT, "snntc_fc_forward_workspace_bytes: bad argument");
    *bytes = fc_fwd_ws(nullptr, B, I).bytes;
    return SNNTC_OK;
}

// Slices of the one-launch backward pass for dense layers with few outputs; 0 when the layer takes
// the general path.  Decided by the layer's shape alone.
static int fc_narrow_split(int64_t B, int64_t I, int64_t J) {
    return (I >= 1 && B >= 1 && fc_backward_narrow_supported(J)) ? fc_backward_narrow_splits(B) : 0;
}

int snntc_fc_backward_workspace_bytes(int64_t B, int64_t I, int64_t J, size_t* bytes) {
    if (!bytes || B < 0 || I < 0 || J < 0)
        return fail(SNNTC_ERR_BAD_ARGUMENT, "snntc_fc_backward_workspace_bytes: bad argument");
    *bytes = bwd_ws(nullptr, B, I + 1, J, grad_weight_blocks(I, J), 0, fc_narrow_split(B, I, J)).bytes;
    return SNNTC_OK;
}

int snntc_fc_forward(const float* x, const float* w, const float* params_host, float* out, int64_t B,
                     int64_t I, int64_t J, int64_t w_rows, void* workspace, size_t workspace_bytes,
                     void* stream) {
    return fc_forward_impl(x, w, params_host, out, nullptr, nullptr, nullptr, B, I, J, w_rows, workspace,
                           workspace_bytes, stream);
}

int snntc_fc_forward_ex(const float* x, const float* w, const float* params_host, float* out,
                        float* sorted_z, int32_t* perm, int32_t* causal_k, int64_t B, int64_t I, int64_t J,
                        int64_t w_rows, void* workspace, size_t workspace_bytes, void* stream) {
    return fc_forward_impl(x, w, params_host, out, sorted_z, perm, causal_k, B, I, J, w_rows, workspace,
                           workspace_bytes, stream);
}

int snntc_init(int device) {
    int current = 0;
    SNNTC_HIP_CHECK(hipGetDevice(&current));
    if (device < 0 || device == current) return prepare_device(current, nullptr);
    SNNTC_HIP_CHECK(hipSetDevice(device));                 // the set-up needs its device current
    const int rc = prepare_device(device, nullptr);
    SNNTC_HIP_CHECK(hipSetDevice(current));
    return rc;
}

size_t snntc_static_scratch_bytes(void) { return kStaticScratchBytes; }

int snntc_fc_forward_static(const float* x, const float* w, const float* params_host, float* out, int64_t B,
                            int64_t I, int64_t J, int64_t w_rows, void* stream) {
    int rc = fc_check(B, I, J, w_rows, params_host, "snntc_fc_forward_static");
    if (rc) return rc;
    const size_t need = fc_fwd_ws(nullptr, B, I).bytes;
    if (need > kStaticScratchBytes)
        return fail(SNNTC_ERR_WORKSPACE,
                    "snntc_fc_forward_static: B=%lld, I=%lld needs %zu bytes of scratch, the library holds %zu "
                    "(use snntc_fc_forward with a workspace of your own)",
                    (long long)B, (long long)I, need, kStaticScratchBytes);
    int dev = 0;
    SNNTC_HIP_CHECK(hipGetDevice(&dev));
    void* ws = nullptr;
    rc = prepare_device(dev, &ws);           // first call on a device: look up this device's copy of the array
    if (rc) return rc;
    // every byte of the workspace the scan reads is written by the sort of this call (padding entries
    // of the rows included), so nothing needs clearing between calls
    return fc_forward_impl(x, w, params_host, out, nullptr, nullptr, nullptr, B, I, J, w_rows, ws,
                           kStaticScratchBytes, stream);
}

int snntc_fc_backward(const float* grad, const float* x, const float* w, const float* params_host,
                      const float* oldout, float* dx, float* dw, float* dparams, int64_t B, int64_t I,
                      int64_t J, int64_t w_rows, int64_t grad_rows, void* workspace, size_t workspace_bytes,
                      void* stream) {
    int rc = fc_check(B, I, J, w_rows, params_host, "snntc_fc_backward");
    if (rc) return rc;
    if (grad_rows != 2 * B)
        return fail(SNNTC_ERR_DIM_MISMATCH, "snntc_fc_backward: Grad/Oldout batch should be 2 * batch (got %lld for batch %lld)",
                    (long long)grad_rows, (long long)B);
    hipStream_t st = static_cast<hipStream_t>(stream);
    // dparams is all zeros; where a backward launch follows, its first workgroup writes them
    if (!dx && !dw) return dparams ? launch_fill_zero(dparams, 6, st) : SNNTC_OK;   // a NULL gradient output is simply not computed
    if (B == 0 || J == 0) {
        if (dparams) { rc = launch_fill_zero(dparams, 6, st); if (rc) return rc; }
        if (dx) { rc = launch_fill_zero(dx, B * I, st); if (rc) return rc; }
        return dw ? launch_fill_zero(dw, w_rows * J, st) : SNNTC_OK;
    }
    if (!grad || !x || !w || !oldout) return fail(SNNTC_ERR_BAD_ARGUMENT, "snntc_fc_backward: NULL tensor pointer");
    const int narrow = fc_narrow_split(B, I, J);
    BwdWs ws = bwd_ws(workspace, B, I + 1, J, grad_weight_blocks(I, J), 0, narrow);
    rc = check_workspace(workspace, workspace_bytes, ws.bytes);
    if (rc) return rc;
    const NeuronParams np = neuron_params(params_host[0], params_host[2], params_host[5]);
    if (narrow)                                          // a classifier head: everything in one launch
        return launch_fc_backward_narrow(x, w, grad, oldout, oldout + B * J, dx, dw, ws.partial, dparams, 6, B, I, J,
                                         np, st);
    // wt[J, I] for dX (the bias row is not needed) is written by the same launch
    rc = launch_backward_prologue(grad, oldout, oldout + B * J, ws.upm, B * J, np, dx ? 1 : 0, w, ws.wt, I, J,
                                  0, dparams, 6, st);
    if (rc) return rc;
    if (dx) {
        rc = launch_fc_grad_input(x, ws.wt, ws.upm, oldout, dx, B, I, J, I, st);
        if (rc) return rc;
    }
    if (!dw) return SNNTC_OK;
    SegmentSource src{};
    src.base = x; src.conv = 0; src.I = (int)I;
    int nsplit = weight_grad_splits(B, grad_weight_blocks(w_rows, J));
    if (nsplit > ws.max_split) nsplit = ws.max_split;
    rc = launch_grad_weight_rows(src, ws.upm, oldout, nsplit > 1 ? ws.partial : dw, nsplit, B, J, 0, np, st);
    if (rc) return rc;
    return launch_reduce_partials(ws.partial, dw, w_rows * J, nsplit, st);
}

int snntc_cv_output_dims(int64_t H, int64_t W, const float* params_host, int64_t* Nh, int64_t* Nw) {
    ConvGeom g;
    int rc = cv_geom(0, H, W, 1, 0, 0, params_host, false, "snntc_cv_output_dims", &g);
    if (rc) return rc;
    if (Nh) *Nh = g.Nh;
    if (Nw) *Nw = g.Nw;
    return SNNTC_OK;
}

int snntc_cv_forward_workspace_bytes(int64_t B, int64_t H, int64_t W, int64_t C, int64_t Kc,
                                     const float* params_host, size_t* bytes) {
    ConvGeom g;
    int rc = cv_geom(B, H, W, C, Kc, 0, params_host, false, "snntc_cv_forward_workspace_bytes", &g);
    if (rc) return rc;
    if (!bytes) return fail(SNNTC_ERR_BAD_ARGUMENT, "snntc_cv_forward_workspace_bytes: bytes is NULL");
    const bool merge = merge_sort_supported(g);
    *bytes = fc_fwd_ws(nullptr, g.S, g.P, merge ? B * H * W : 0, merge ? C : 0).bytes;
    return SNNTC_OK;
}

int snntc_cv_backward_workspace_bytes(int64_t B, int64_t H, int64_t W, int64_t C, int64_t Kc,
                                      const float* params_host, size_t* bytes) {
    ConvGeom g;
    int rc = cv_geom(B, H, W, C, Kc, 0, params_host, false, "snntc_cv_backward_workspace_bytes", &g);
    if (rc) return rc;
    if (!bytes) return fail(SNNTC_ERR_BAD_ARGUMENT, "snntc_cv_backward_workspace_bytes: bytes is NULL");
    *bytes = bwd_ws(nullptr, g.S, g.P + 1, Kc, cv_weight_base_blocks(g),
                    cv_grad_input_chan_supported(g) ? 0 : g.S * g.P).bytes;
    return SNNTC_OK;
}

int snntc_cv_forward(const float* xpad, const float* w, const float* params_host, float* out, int64_t B,
                     int64_t H, int64_t W, int64_t C, int64_t Kc, int64_t w_rows, void* workspace,
                     size_t workspace_bytes, void* stream) {
    return cv_forward_impl(xpad, w, params_host, out, nullptr, nullptr, nullptr, nullptr, 0, 0, 0, 0, B, H, W, C, Kc,
                           w_rows, workspace, workspace_bytes, stream);
}

int snntc_cv_forward_chained(const float* xpad, const float* w, const float* params_host, float* out,
                             float* next_xpad, int64_t next_h, int64_t next_w, int64_t next_top, int64_t next_left,
                             int64_t B, int64_t H, int64_t W, int64_t C, int64_t Kc, int64_t w_rows,
                             void* workspace, size_t workspace_bytes, void* stream) {
    if (!next_xpad) return fail(SNNTC_ERR_BAD_ARGUMENT, "snntc_cv_forward_chained: next_xpad is NULL");
    return cv_forward_impl(xpad, w, params_host, out, nullptr, nullptr, nullptr, next_xpad, next_h, next_w, next_top,
                           next_left, B, H, W, C, Kc, w_rows, workspace, workspace_bytes, stream);
}

int snntc_cv_forward_ex(const float* xpad, const float* w, const float* params_host, float* out,
                        float* sorted_z, int32_t* perm, int32_t* causal_k, int64_t B, int64_t H, int64_t W,
                        int64_t C, int64_t Kc, int64_t w_rows, void* workspace, size_t workspace_bytes,
                        void* stream) {
    return cv_forward_impl(xpad, w, params_host, out, sorted_z, perm, causal_k, nullptr, 0, 0, 0, 0, B, H, W, C, Kc,
                           w_rows, workspace, workspace_bytes, stream);
}

// dx[B, crop.h, crop.w, C]: the window of the padded input's gradient that starts at (crop.top, crop.left)
static int cv_backward_impl(const float* grad, const float* xpad, const float* w, const float* params_host,
                            const float* oldout, float* dxpad, CropGeom crop, float* dw, float* dparams, int64_t B,
                            int64_t H, int64_t W, int64_t C, int64_t Kc, int64_t w_rows, int64_t grad_rows,
                            void* workspace, size_t workspace_bytes, void* stream) {
    ConvGeom g;
    int rc = cv_geom(B, H, W, C, Kc, w_rows, params_host, true, "snntc_cv_backward", &g);
    if (rc) return rc;
    if (grad_rows != 2 * B)
        return fail(SNNTC_ERR_DIM_MISMATCH, "snntc_cv_backward: Grad/Oldout batch should be 2 * batch (got %lld for batch %lld)",
                    (long long)grad_rows, (long long)B);
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (!dxpad && !dw) return dparams ? launch_fill_zero(dparams, 12, st) : SNNTC_OK;   // a NULL gradient output is simply not computed
    if (g.S == 0 || Kc == 0) {
        if (dparams) { rc = launch_fill_zero(dparams, 12, st); if (rc) return rc; }
        if (dxpad) { rc = launch_fill_zero(dxpad, B * crop.h * crop.w * C, st); if (rc) return rc; }
        return dw ? launch_fill_zero(dw, w_rows * Kc, st) : SNNTC_OK;
    }
    if (!grad || !xpad || !w || !oldout) return fail(SNNTC_ERR_BAD_ARGUMENT, "snntc_cv_backward: NULL tensor pointer");
    BwdWs ws = bwd_ws(workspace, g.S, g.P + 1, Kc, cv_weight_base_blocks(g),
                      cv_grad_input_chan_supported(g) ? 0 : g.S * g.P);
    rc = check_workspace(workspace, workspace_bytes, ws.bytes);
    if (rc) return rc;
    const NeuronParams np = neuron_params(params_host[0], params_host[4], params_host[11]);
    // the weight copy dX reads from is written by the same launch: regrouped for the channel kernel,
    // wt[Kc, P] for the generic one
    const bool chan_dx = cv_grad_input_chan_supported(g);
    rc = launch_backward_prologue(grad, oldout, oldout + g.S * Kc, ws.upm, g.S * Kc, np,
                                  !dxpad ? 0 : chan_dx ? 2 : 1, w, ws.wt, g.P, Kc, g.C, dparams, 12, st);
    if (rc) return rc;
    if (dxpad) {
        if (chan_dx) {
            rc = launch_cv_grad_input_chan(xpad, ws.wt, ws.upm, oldout, dxpad, crop, g, np, st);
        } else {
            rc = launch_cv_grad_input(conv_source(xpad, g), ws.wt, ws.upm, oldout, ws.dxp, dxpad, crop, g, g.P, st);
        }
        if (rc) return rc;
    }
    if (!dw) return SNNTC_OK;
    const bool wide = cv_grad_weight_wide_supported(g);
    int nsplit = weight_grad_splits(g.S, wide ? cv_grad_weight_wide_blocks(g) : grad_weight_blocks(w_rows, Kc));
    if (nsplit > ws.max_split) nsplit = ws.max_split;
    float* dst = nsplit > 1 ? ws.partial : dw;
    const SegmentSource src = conv_source(xpad, g);
    if (wide) {
        rc = launch_cv_grad_weight_wide(xpad, ws.upm, oldout, dst, nsplit, g, w_rows, np, st);
    } else {
        rc = launch_grad_weight_rows(src, ws.upm, oldout, dst, nsplit, g.S, Kc, 0, np, st);
    }
    if (rc) return rc;
    return launch_reduce_partials(ws.partial, dw, w_rows * Kc, nsplit, st);
}

int snntc_cv_backward(const float* grad, const float* xpad, const float* w, const float* params_host,
                      const float* oldout, float* dxpad, float* dw, float* dparams, int64_t B, int64_t H,
                      int64_t W, int64_t C, int64_t Kc, int64_t w_rows, int64_t grad_rows, void* workspace,
                      size_t workspace_bytes, void* stream) {
    return cv_backward_impl(grad, xpad, w, params_host, oldout, dxpad, CropGeom{(int)H, (int)W, 0, 0}, dw, dparams, B,
                            H, W, C, Kc, w_rows, grad_rows, workspace, workspace_bytes, stream);
}

int snntc_cv_backward_cropped(const float* grad, const float* xpad, const float* w, const float* params_host,
                              const float* oldout, float* dx, int64_t dx_h, int64_t dx_w, int64_t dx_top,
                              int64_t dx_left, float* dw, float* dparams, int64_t B, int64_t H, int64_t W, int64_t C,
                              int64_t Kc, int64_t w_rows, int64_t grad_rows, void* workspace, size_t workspace_bytes,
                              void* stream) {
    if (dx_h < 0 || dx_w < 0 || dx_top < 0 || dx_left < 0 || dx_top + dx_h > H || dx_left + dx_w > W)
        return fail(SNNTC_ERR_BAD_ARGUMENT, "snntc_cv_backward_cropped: the %lld x %lld window at (%lld, %lld) does not "
                    "lie inside the %lld x %lld padded image", (long long)dx_h, (long long)dx_w, (long long)dx_top,
                    (long long)dx_left, (long long)H, (long long)W);
    return cv_backward_impl(grad, xpad, w, params_host, oldout, dx,
                            CropGeom{(int)dx_h, (int)dx_w, (int)dx_top, (int)dx_left}, dw, dparams, B, H, W, C, Kc,
                            w_rows, grad_rows, workspace, workspace_bytes, stream);
}

}  // extern "C"
