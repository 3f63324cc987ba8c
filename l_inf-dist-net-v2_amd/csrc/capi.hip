// extern "C" entry points of libnorm_dist_hip.so: argument validation, geometry, dispatch to the kernel launchers.
// One function per member of the reference's kernel interface (core/cuda/norm_dist.h:4-38); the checks mirror
// what the reference's binding layer enforces (core/cuda/norm_dist.cpp:8-12) as far as raw pointers allow.
#include "../../include/norm_dist_hip.h"

#include <algorithm>
#include <atomic>
#include <cmath>
#include <mutex>

#include "ndist_common.h"

namespace ndist {

static thread_local int g_last_hip_error = 0;

bool hip_failed(hipError_t e) {
    if (e == hipSuccess) return false;
    g_last_hip_error = (int)e;
    (void)hipGetLastError();  // clear the sticky launch error so that later calls are not blamed for it
    return true;
}

int hip_status(hipError_t e) {
    if (!hip_failed(e)) return NDIST_OK;
    if (e == hipErrorStreamCaptureUnsupported) return NDIST_ERR_CAPTURE;
    if (e == hipErrorOutOfMemory && static_scratch_active()) return NDIST_ERR_TOO_LARGE;
    return NDIST_ERR_HIP;
}

namespace {
constexpr int kMaxDev = 64;
DeviceInfo g_di_cache[kMaxDev];
bool g_di_have[kMaxDev] = {};
std::mutex g_di_mu;
}  // namespace

bool device_info_cached() {
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDev) dev = 0;
    std::lock_guard<std::mutex> lock(g_di_mu);
    return g_di_have[dev];
}

const DeviceInfo& device_info() {
    DeviceInfo* cache = g_di_cache;
    bool* have = g_di_have;
    std::mutex& mu = g_di_mu;
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDev) dev = 0;
    std::lock_guard<std::mutex> lock(mu);
    if (!have[dev]) {
        hipDeviceProp_t prop;
        DeviceInfo di{256, 160 * 1024};
        if (hipGetDeviceProperties(&prop, dev) == hipSuccess) {
            di.num_cu = prop.multiProcessorCount > 0 ? prop.multiProcessorCount : 256;
            di.lds_bytes = (int)prop.sharedMemPerBlock;
        }
        cache[dev] = di;
        have[dev] = true;
    }
    return cache[dev];
}

static std::atomic<int> g_profiling{0};
// The timing state is process-wide, not per thread: frameworks run the backward on a worker thread while the
// caller reads the result from its own.  Profiling is a single-caller measurement aid; concurrent profiled calls
// simply overwrite each other's events.
static hipEvent_t g_ev_start = nullptr, g_ev_stop = nullptr;
static std::atomic<bool> g_ev_valid{false};
static thread_local int g_timer_depth = 0;  // nested timers: only the outermost records
static std::mutex g_ev_mu;

KernelTimer::KernelTimer(hipStream_t st) : stream(st), active(g_profiling.load(std::memory_order_relaxed) != 0) {
    if (!active) return;
    // no event records into a graph under capture, and nothing that allocates inside the no-allocation entry point
    if (static_scratch_active() || stream_is_capturing(st)) {
        active = false;
        return;
    }
    if (g_timer_depth++ > 0) return;
    std::lock_guard<std::mutex> lock(g_ev_mu);
    if (g_ev_start == nullptr) {
        if (hipEventCreate(&g_ev_start) != hipSuccess || hipEventCreate(&g_ev_stop) != hipSuccess) {
            g_timer_depth--;
            active = false;
            return;
        }
    }
    g_ev_valid = false;
    (void)hipEventRecord(g_ev_start, stream);
}
KernelTimer::~KernelTimer() {
    if (!active) return;
    if (--g_timer_depth > 0) return;
    std::lock_guard<std::mutex> lock(g_ev_mu);
    g_ev_valid = hipEventRecord(g_ev_stop, stream) == hipSuccess;
}

static int make_geom(int B, int CO, int CI, int G, int HW, Geom* out) {
    if (B <= 0 || CO <= 0 || CI <= 0 || G <= 0 || HW <= 0) return NDIST_ERR_BAD_SHAPE;
    if (CI % G != 0 || CO % G != 0) return NDIST_ERR_BAD_SHAPE;
    const long long lim = 0x7fffffffLL;
    if ((long long)B * HW > lim || (long long)B * HW * CO > lim || (long long)B * HW * CI > lim ||
        (long long)CO * (CI / G) > lim)
        return NDIST_ERR_BAD_SHAPE;
    out->B = B;
    out->HW = HW;
    out->M = B * HW;
    out->COg = CO / G;
    out->CIg = CI / G;
    out->G = G;
    return NDIST_OK;
}

static int make_unfold_geom(int B, int C, int H, int W, int kh, int kw, int dh, int dw, int ph, int pw, int sh, int sw,
                            UnfoldGeom* u) {
    if (B <= 0 || C <= 0 || H <= 0 || W <= 0 || kh <= 0 || kw <= 0 || dh <= 0 || dw <= 0 || ph < 0 || pw < 0 || sh <= 0 ||
        sw <= 0)
        return NDIST_ERR_BAD_SHAPE;
    const long long eh = (long long)H + 2LL * ph - (long long)dh * (kh - 1) - 1;
    const long long ew = (long long)W + 2LL * pw - (long long)dw * (kw - 1) - 1;
    if (eh < 0 || ew < 0) return NDIST_ERR_BAD_SHAPE;
    const long long OH = eh / sh + 1, OW = ew / sw + 1;
    const long long lim = 0x7fffffffLL;
    if ((long long)B * C * H * W > lim || OH * OW > lim || (long long)C * kh * kw > lim ||
        (long long)B * C * kh * kw * OH * OW > 4 * lim)
        return NDIST_ERR_BAD_SHAPE;
    *u = UnfoldGeom{B, C, H, W, kh, kw, dh, dw, ph, pw, sh, sw, (int)OH, (int)OW};
    return NDIST_OK;
}

static bool finite_positive(float p) { return p > 0.0f && std::isfinite(p); }

}  // namespace ndist

using namespace ndist;

#define NDIST_REQUIRE(ptr) \
    if ((ptr) == nullptr) return NDIST_ERR_NULL_POINTER

extern "C" {

int ndist_version(void) { return 10000; }

const char* ndist_status_string(int status) {
    switch (status) {
        case NDIST_OK: return "success";
        case NDIST_ERR_NULL_POINTER: return "a required pointer is NULL";
        case NDIST_ERR_BAD_SHAPE: return "invalid shape (non-positive size, channels not divisible by groups, or too large)";
        case NDIST_ERR_BAD_P: return "p must be positive and finite";
        case NDIST_ERR_HIP: return "a HIP runtime call failed";
        case NDIST_ERR_NO_DEVICE: return "no usable HIP device";
        case NDIST_ERR_CAPTURE: return "the stream is being captured into a graph and this call needs temporary device memory";
        case NDIST_ERR_TOO_LARGE: return "the problem needs more temporary device memory than the fixed scratch array holds";
        default: return "unknown status";
    }
}

int ndist_last_hip_error(void) { return g_last_hip_error; }

void ndist_set_profiling(int enable) { g_profiling.store(enable ? 1 : 0); }

void ndist_set_skip_mode(int skip, int bounds) { set_skip_mode(skip, bounds); }
void ndist_set_hot_mode(int mode) { set_hot_mode(mode); }
void ndist_set_scaled_mode(int mode) { set_scaled_mode(mode); }
void ndist_get_modes(int* skip, int* bounds, int* hot, int* scaled) {
    int s = -1, b = -1;
    get_skip_mode(&s, &b);
    if (skip != nullptr) *skip = s;
    if (bounds != nullptr) *bounds = b;
    if (hot != nullptr) *hot = hot_mode();
    if (scaled != nullptr) *scaled = scaled_mode();
}

int ndist_release_scratch(void) { return scratch_release_all(); }

void ndist_scratch_counters(long* mallocs, long* frees) {
    long m = 0, f = 0;
    scratch_counters(&m, &f);
    if (mallocs != nullptr) *mallocs = m;
    if (frees != nullptr) *frees = f;
}

size_t ndist_noalloc_scratch_bytes(void) { return kStaticScratchBytes; }

int ndist_noalloc_prepare(void) {
    char* base = nullptr;
    if (int rc = hip_status(static_scratch_base(&base, true))) return rc;
    (void)device_info();
    return device_info_cached() ? NDIST_OK : NDIST_ERR_NO_DEVICE;
}

int ndist_last_kernel_ms(float* ms) {
    if (ms == nullptr) return NDIST_ERR_NULL_POINTER;
    if (!g_ev_valid) return NDIST_ERR_BAD_SHAPE;
    std::lock_guard<std::mutex> lock(g_ev_mu);
    NDIST_HIP_TRY(hipEventSynchronize(g_ev_stop));
    NDIST_HIP_TRY(hipEventElapsedTime(ms, g_ev_start, g_ev_stop));
    return NDIST_OK;
}

int ndist_norm_dist_forward(const float* input, const float* weight, int B, int CO, int CI, int G, int HW, float* output,
                            float p, ndist_stream_t stream) {
    NDIST_REQUIRE(input); NDIST_REQUIRE(weight); NDIST_REQUIRE(output);
    if (!finite_positive(p)) return NDIST_ERR_BAD_P;
    Geom s;
    if (int rc = make_geom(B, CO, CI, G, HW, &s)) return rc;
    return launch_norm_forward(input, weight, nullptr, s, output, p, (hipStream_t)stream);
}

int ndist_norm_dist_forward_with_max(const float* input, const float* weight, const float* max_output, int B, int CO,
                                     int CI, int G, int HW, float* output, float p, ndist_stream_t stream) {
    NDIST_REQUIRE(input); NDIST_REQUIRE(weight); NDIST_REQUIRE(max_output); NDIST_REQUIRE(output);
    if (!finite_positive(p)) return NDIST_ERR_BAD_P;
    Geom s;
    if (int rc = make_geom(B, CO, CI, G, HW, &s)) return rc;
    return launch_norm_forward(input, weight, max_output, s, output, p, (hipStream_t)stream);
}

int ndist_norm_dist_backward_input(const float* grad_output, const float* input, const float* weight,
                                   const float* output, int B, int CO, int CI, int G, int HW, float* grad_input, float p,
                                   ndist_stream_t stream) {
    NDIST_REQUIRE(grad_output); NDIST_REQUIRE(input); NDIST_REQUIRE(weight); NDIST_REQUIRE(output);
    NDIST_REQUIRE(grad_input);
    if (!finite_positive(p)) return NDIST_ERR_BAD_P;
    Geom s;
    if (int rc = make_geom(B, CO, CI, G, HW, &s)) return rc;
    return launch_norm_backward(grad_output, input, weight, output, s, grad_input, nullptr, p, (hipStream_t)stream);
}

int ndist_norm_dist_backward_input_weight(const float* grad_output, const float* input, const float* weight,
                                          const float* output, int B, int CO, int CI, int G, int HW, float* grad_input,
                                          float* grad_weight, float p, ndist_stream_t stream) {
    NDIST_REQUIRE(grad_output); NDIST_REQUIRE(input); NDIST_REQUIRE(weight); NDIST_REQUIRE(output);
    NDIST_REQUIRE(grad_input); NDIST_REQUIRE(grad_weight);
    if (!finite_positive(p)) return NDIST_ERR_BAD_P;
    Geom s;
    if (int rc = make_geom(B, CO, CI, G, HW, &s)) return rc;
    return launch_norm_backward(grad_output, input, weight, output, s, grad_input, grad_weight, p, (hipStream_t)stream);
}

int ndist_norm_dist_backward_input_weight_noalloc(const float* grad_output, const float* input, const float* weight,
                                                  const float* output, int B, int CO, int CI, int G, int HW,
                                                  float* grad_input, float* grad_weight, float p,
                                                  ndist_stream_t stream) {
    NDIST_REQUIRE(grad_output); NDIST_REQUIRE(input); NDIST_REQUIRE(weight); NDIST_REQUIRE(output);
    NDIST_REQUIRE(grad_input); NDIST_REQUIRE(grad_weight);
    if (!finite_positive(p)) return NDIST_ERR_BAD_P;
    Geom s;
    if (int rc = make_geom(B, CO, CI, G, HW, &s)) return rc;
    // the factor array is the one piece of scratch the kernels cannot do without: refuse before anything is launched
    if (norm_backward_scratch_bytes(s, p) > kStaticScratchBytes) return NDIST_ERR_TOO_LARGE;
    // scratch_alloc serves from the fixed array while the scope lives.  The array's address and the device's
    // properties are looked up once per device: by ndist_noalloc_prepare() or by the first call outside a capture;
    // a call on a capturing stream that finds them missing refuses instead of querying the runtime mid-capture.
    const bool capturing = stream_is_capturing((hipStream_t)stream);
    if (capturing && !device_info_cached()) return NDIST_ERR_CAPTURE;
    StaticScratchScope scope(!capturing);
    if (scope.status == hipErrorStreamCaptureUnsupported) return NDIST_ERR_CAPTURE;
    if (int rc = hip_status(scope.status)) return rc;
    return launch_norm_backward(grad_output, input, weight, output, s, grad_input, grad_weight, p, (hipStream_t)stream);
}

int ndist_inf_dist_forward_nograd(const float* input, const float* weight, int B, int CO, int CI, int G, int HW,
                                  float* output, ndist_stream_t stream) {
    NDIST_REQUIRE(input); NDIST_REQUIRE(weight); NDIST_REQUIRE(output);
    Geom s;
    if (int rc = make_geom(B, CO, CI, G, HW, &s)) return rc;
    return launch_inf_forward(input, weight, s, output, nullptr, (hipStream_t)stream);
}

int ndist_inf_dist_forward(const float* input, const float* weight, int B, int CO, int CI, int G, int HW, float* output,
                           int32_t* pos, ndist_stream_t stream) {
    NDIST_REQUIRE(input); NDIST_REQUIRE(weight); NDIST_REQUIRE(output); NDIST_REQUIRE(pos);
    Geom s;
    if (int rc = make_geom(B, CO, CI, G, HW, &s)) return rc;
    return launch_inf_forward(input, weight, s, output, pos, (hipStream_t)stream);
}

int ndist_inf_dist_backward_input(const float* grad_output, const int32_t* pos, int B, int CO, int CI, int G, int HW,
                                  float* grad_input, ndist_stream_t stream) {
    NDIST_REQUIRE(grad_output); NDIST_REQUIRE(pos); NDIST_REQUIRE(grad_input);
    Geom s;
    if (int rc = make_geom(B, CO, CI, G, HW, &s)) return rc;
    return launch_inf_backward(grad_output, pos, s, grad_input, nullptr, (hipStream_t)stream);
}

int ndist_inf_dist_backward_input_weight(const float* grad_output, const int32_t* pos, int B, int CO, int CI, int G,
                                         int HW, float* grad_input, float* grad_weight, ndist_stream_t stream) {
    NDIST_REQUIRE(grad_output); NDIST_REQUIRE(pos); NDIST_REQUIRE(grad_input); NDIST_REQUIRE(grad_weight);
    Geom s;
    if (int rc = make_geom(B, CO, CI, G, HW, &s)) return rc;
    return launch_inf_backward(grad_output, pos, s, grad_input, grad_weight, (hipStream_t)stream);
}

int ndist_bound_inf_dist_forward_nograd(const float* inputL, const float* inputU, const float* weight, int B, int CO,
                                        int CI, int G, int HW, float* outputL, float* outputU, ndist_stream_t stream) {
    NDIST_REQUIRE(inputL); NDIST_REQUIRE(inputU); NDIST_REQUIRE(weight); NDIST_REQUIRE(outputL); NDIST_REQUIRE(outputU);
    Geom s;
    if (int rc = make_geom(B, CO, CI, G, HW, &s)) return rc;
    return launch_bound_forward(inputL, inputU, weight, s, outputL, outputU, nullptr, nullptr, (hipStream_t)stream);
}

int ndist_bound_inf_dist_forward(const float* inputL, const float* inputU, const float* weight, int B, int CO, int CI,
                                 int G, int HW, float* outputL, float* outputU, int32_t* posL, int32_t* posU,
                                 ndist_stream_t stream) {
    NDIST_REQUIRE(inputL); NDIST_REQUIRE(inputU); NDIST_REQUIRE(weight); NDIST_REQUIRE(outputL); NDIST_REQUIRE(outputU);
    NDIST_REQUIRE(posL); NDIST_REQUIRE(posU);
    Geom s;
    if (int rc = make_geom(B, CO, CI, G, HW, &s)) return rc;
    return launch_bound_forward(inputL, inputU, weight, s, outputL, outputU, posL, posU, (hipStream_t)stream);
}

int ndist_bound_inf_dist_backward_input(const float* grad_outputL, const float* grad_outputU, const int32_t* posL,
                                        const int32_t* posU, int B, int CO, int CI, int G, int HW, float* grad_inputL,
                                        float* grad_inputU, ndist_stream_t stream) {
    NDIST_REQUIRE(grad_outputL); NDIST_REQUIRE(grad_outputU); NDIST_REQUIRE(posL); NDIST_REQUIRE(posU);
    NDIST_REQUIRE(grad_inputL); NDIST_REQUIRE(grad_inputU);
    Geom s;
    if (int rc = make_geom(B, CO, CI, G, HW, &s)) return rc;
    return launch_bound_backward(grad_outputL, grad_outputU, posL, posU, s, grad_inputL, grad_inputU, nullptr,
                                 (hipStream_t)stream);
}

int ndist_bound_inf_dist_backward_input_weight(const float* grad_outputL, const float* grad_outputU,
                                               const int32_t* posL, const int32_t* posU, int B, int CO, int CI, int G,
                                               int HW, float* grad_inputL, float* grad_inputU, float* grad_weight,
                                               ndist_stream_t stream) {
    NDIST_REQUIRE(grad_outputL); NDIST_REQUIRE(grad_outputU); NDIST_REQUIRE(posL); NDIST_REQUIRE(posU);
    NDIST_REQUIRE(grad_inputL); NDIST_REQUIRE(grad_inputU); NDIST_REQUIRE(grad_weight);
    Geom s;
    if (int rc = make_geom(B, CO, CI, G, HW, &s)) return rc;
    return launch_bound_backward(grad_outputL, grad_outputU, posL, posU, s, grad_inputL, grad_inputU, grad_weight,
                                 (hipStream_t)stream);
}

int ndist_inf_and_bound_forward_nograd(const float* input, const float* inputL, const float* inputU, const float* weight,
                                       int B, int CO, int CI, int G, int HW, float* output, float* outputL,
                                       float* outputU, ndist_stream_t stream) {
    NDIST_REQUIRE(input); NDIST_REQUIRE(inputL); NDIST_REQUIRE(inputU); NDIST_REQUIRE(weight);
    NDIST_REQUIRE(output); NDIST_REQUIRE(outputL); NDIST_REQUIRE(outputU);
    Geom s;
    if (int rc = make_geom(B, CO, CI, G, HW, &s)) return rc;
    return launch_inf_bound_forward(input, inputL, inputU, weight, s, output, nullptr, outputL, outputU, nullptr, nullptr,
                                    (hipStream_t)stream);
}

int ndist_inf_and_bound_forward(const float* input, const float* inputL, const float* inputU, const float* weight, int B,
                                int CO, int CI, int G, int HW, float* output, int32_t* pos, float* outputL,
                                float* outputU, int32_t* posL, int32_t* posU, ndist_stream_t stream) {
    NDIST_REQUIRE(input); NDIST_REQUIRE(inputL); NDIST_REQUIRE(inputU); NDIST_REQUIRE(weight);
    NDIST_REQUIRE(output); NDIST_REQUIRE(outputL); NDIST_REQUIRE(outputU);
    NDIST_REQUIRE(pos); NDIST_REQUIRE(posL); NDIST_REQUIRE(posU);
    Geom s;
    if (int rc = make_geom(B, CO, CI, G, HW, &s)) return rc;
    return launch_inf_bound_forward(input, inputL, inputU, weight, s, output, pos, outputL, outputU, posL, posU,
                                    (hipStream_t)stream);
}

long long ndist_weight_cache_bytes(int CO, int CI, int G) {
    Geom s;
    if (make_geom(1, CO, CI, G, 1, &s)) return 0;
    return (long long)(weight_seed_floats(s) * sizeof(float));
}

int ndist_weight_cache_prepare(const float* weight, int CO, int CI, int G, void* cache, ndist_stream_t stream) {
    NDIST_REQUIRE(weight); NDIST_REQUIRE(cache);
    Geom s;
    if (int rc = make_geom(1, CO, CI, G, 1, &s)) return rc;
    WeightSeeds ws{};
    return launch_weight_seeds(weight, s, static_cast<float*>(cache), nullptr, 0, (hipStream_t)stream, &ws);
}

int ndist_inf_dist_forward_nograd_cached(const float* input, const float* weight, const void* cache, int B, int CO, int CI,
                                         int G, int HW, float* output, ndist_stream_t stream) {
    NDIST_REQUIRE(input); NDIST_REQUIRE(weight); NDIST_REQUIRE(cache); NDIST_REQUIRE(output);
    Geom s;
    if (int rc = make_geom(B, CO, CI, G, HW, &s)) return rc;
    const WeightSeeds ws = weight_seeds_at(static_cast<float*>(const_cast<void*>(cache)), s);
    return launch_inf_forward(input, weight, s, output, nullptr, (hipStream_t)stream, nullptr, &ws);
}

int ndist_inf_and_bound_forward_nograd_cached(const float* input, const float* inputL, const float* inputU,
                                              const float* weight, const void* cache, int B, int CO, int CI, int G, int HW,
                                              float* output, float* outputL, float* outputU, ndist_stream_t stream) {
    NDIST_REQUIRE(input); NDIST_REQUIRE(inputL); NDIST_REQUIRE(inputU); NDIST_REQUIRE(weight); NDIST_REQUIRE(cache);
    NDIST_REQUIRE(output); NDIST_REQUIRE(outputL); NDIST_REQUIRE(outputU);
    Geom s;
    if (int rc = make_geom(B, CO, CI, G, HW, &s)) return rc;
    const WeightSeeds ws = weight_seeds_at(static_cast<float*>(const_cast<void*>(cache)), s);
    return launch_inf_bound_forward(input, inputL, inputU, weight, s, output, nullptr, outputL, outputU, nullptr, nullptr,
                                    (hipStream_t)stream, &ws);
}

int ndist_unfold_forward(const float* input, int B, int C, int H, int W, int kernel_h, int kernel_w, int dilation_h,
                         int dilation_w, int padding_h, int padding_w, int stride_h, int stride_w, float* output,
                         ndist_stream_t stream) {
    NDIST_REQUIRE(input); NDIST_REQUIRE(output);
    UnfoldGeom u;
    if (int rc = make_unfold_geom(B, C, H, W, kernel_h, kernel_w, dilation_h, dilation_w, padding_h, padding_w, stride_h,
                                  stride_w, &u))
        return rc;
    return launch_unfold(input, u, output, (hipStream_t)stream);
}

int ndist_unfold_backward(const float* grad_output, int B, int C, int H, int W, int kernel_h, int kernel_w,
                          int dilation_h, int dilation_w, int padding_h, int padding_w, int stride_h, int stride_w,
                          float* grad_input, ndist_stream_t stream) {
    NDIST_REQUIRE(grad_output); NDIST_REQUIRE(grad_input);
    UnfoldGeom u;
    if (int rc = make_unfold_geom(B, C, H, W, kernel_h, kernel_w, dilation_h, dilation_w, padding_h, padding_w, stride_h,
                                  stride_w, &u))
        return rc;
    return launch_fold(grad_output, u, grad_input, (hipStream_t)stream);
}

// ---- convolutional layer without the unfolded tensor ------------------------------------------------------------
// geometry of the fused calls: the patch geometry, and the distance problem it unfolds to
static int make_conv_geom(int B, int C, int H, int W, int CO, int G, int kh, int kw, int dh, int dw, int ph, int pw,
                          int sh, int sw, UnfoldGeom* u, Geom* s) {
    if (int rc = make_unfold_geom(B, C, H, W, kh, kw, dh, dw, ph, pw, sh, sw, u)) return rc;
    const long long ci = (long long)C * kh * kw, hw = (long long)u->OH * u->OW;
    if (G <= 0 || C % G != 0 || ci / G >= (1 << 22) || u->H >= (1 << 24) || u->W >= (1 << 24)) return NDIST_ERR_BAD_SHAPE;
    return make_geom(B, CO, (int)ci, G, (int)hw, s);
}

int ndist_conv_inf_dist_forward_nograd(const float* input, const float* weight, int B, int C, int H, int W, int CO, int G,
                                       int kernel_h, int kernel_w, int dilation_h, int dilation_w, int padding_h,
                                       int padding_w, int stride_h, int stride_w, float* output, ndist_stream_t stream) {
    NDIST_REQUIRE(input); NDIST_REQUIRE(weight); NDIST_REQUIRE(output);
    UnfoldGeom u;
    Geom s;
    if (int rc = make_conv_geom(B, C, H, W, CO, G, kernel_h, kernel_w, dilation_h, dilation_w, padding_h, padding_w,
                                stride_h, stride_w, &u, &s))
        return rc;
    return launch_inf_forward(input, weight, s, output, nullptr, (hipStream_t)stream, &u);
}

int ndist_conv_bound_inf_dist_forward_nograd(const float* inputL, const float* inputU, const float* weight, int B, int C,
                                             int H, int W, int CO, int G, int kernel_h, int kernel_w, int dilation_h,
                                             int dilation_w, int padding_h, int padding_w, int stride_h, int stride_w,
                                             float* outputL, float* outputU, ndist_stream_t stream) {
    NDIST_REQUIRE(inputL); NDIST_REQUIRE(inputU); NDIST_REQUIRE(weight); NDIST_REQUIRE(outputL); NDIST_REQUIRE(outputU);
    UnfoldGeom u;
    Geom s;
    if (int rc = make_conv_geom(B, C, H, W, CO, G, kernel_h, kernel_w, dilation_h, dilation_w, padding_h, padding_w,
                                stride_h, stride_w, &u, &s))
        return rc;
    return launch_bound_forward(inputL, inputU, weight, s, outputL, outputU, nullptr, nullptr, (hipStream_t)stream, &u);
}

int ndist_conv_inf_dist_forward(const float* input, const float* weight, int B, int C, int H, int W, int CO, int G,
                                int kernel_h, int kernel_w, int dilation_h, int dilation_w, int padding_h, int padding_w,
                                int stride_h, int stride_w, float* output, int32_t* pos, ndist_stream_t stream) {
    NDIST_REQUIRE(input); NDIST_REQUIRE(weight); NDIST_REQUIRE(output); NDIST_REQUIRE(pos);
    UnfoldGeom u;
    Geom s;
    if (int rc = make_conv_geom(B, C, H, W, CO, G, kernel_h, kernel_w, dilation_h, dilation_w, padding_h, padding_w,
                                stride_h, stride_w, &u, &s))
        return rc;
    return launch_inf_forward(input, weight, s, output, pos, (hipStream_t)stream, &u);
}

int ndist_conv_bound_inf_dist_forward(const float* inputL, const float* inputU, const float* weight, int B, int C, int H,
                                      int W, int CO, int G, int kernel_h, int kernel_w, int dilation_h, int dilation_w,
                                      int padding_h, int padding_w, int stride_h, int stride_w, float* outputL,
                                      float* outputU, int32_t* posL, int32_t* posU, ndist_stream_t stream) {
    NDIST_REQUIRE(inputL); NDIST_REQUIRE(inputU); NDIST_REQUIRE(weight); NDIST_REQUIRE(outputL); NDIST_REQUIRE(outputU);
    NDIST_REQUIRE(posL); NDIST_REQUIRE(posU);
    UnfoldGeom u;
    Geom s;
    if (int rc = make_conv_geom(B, C, H, W, CO, G, kernel_h, kernel_w, dilation_h, dilation_w, padding_h, padding_w,
                                stride_h, stride_w, &u, &s))
        return rc;
    return launch_bound_forward(inputL, inputU, weight, s, outputL, outputU, posL, posU, (hipStream_t)stream, &u);
}

// Backward of the fused layer.  The image-gradient kernels need one image plane (and one weight row) in LDS; other
// geometries go the long way: gradient of the unfolded tensor in scratch memory, then the adjoint of
// the patch extraction.
int ndist_conv_norm_dist_forward(const float* input, const float* weight, int B, int C, int H, int W, int CO, int G,
                                 int kernel_h, int kernel_w, int dilation_h, int dilation_w, int padding_h, int padding_w,
                                 int stride_h, int stride_w, float* output, float p, ndist_stream_t stream) {
    NDIST_REQUIRE(input); NDIST_REQUIRE(weight); NDIST_REQUIRE(output);
    if (!finite_positive(p)) return NDIST_ERR_BAD_P;
    UnfoldGeom u;
    Geom s;
    if (int rc = make_conv_geom(B, C, H, W, CO, G, kernel_h, kernel_w, dilation_h, dilation_w, padding_h, padding_w,
                                stride_h, stride_w, &u, &s))
        return rc;
    return launch_norm_forward_conv(input, weight, s, output, p, (hipStream_t)stream, u);
}

static int conv_norm_backward(const float* grad_output, const float* input, const float* weight, const float* output,
                              int B, int C, int H, int W, int CO, int G, int kernel_h, int kernel_w, int dilation_h,
                              int dilation_w, int padding_h, int padding_w, int stride_h, int stride_w, float* grad_input,
                              float* grad_weight, float p, ndist_stream_t stream) {
    NDIST_REQUIRE(grad_output); NDIST_REQUIRE(input); NDIST_REQUIRE(weight); NDIST_REQUIRE(output);
    NDIST_REQUIRE(grad_input);
    if (!finite_positive(p)) return NDIST_ERR_BAD_P;
    UnfoldGeom u;
    Geom s;
    if (int rc = make_conv_geom(B, C, H, W, CO, G, kernel_h, kernel_w, dilation_h, dilation_w, padding_h, padding_w,
                                stride_h, stride_w, &u, &s))
        return rc;
    // The backward's kernel writes gradient rows and, where it does not gather the patches from the images itself
    // (term-skipping variants, tiny batches), reads the patches as rows: one or two buffers of the unfolded size
    // (B x C kh kw x OH OW floats each, 604 MB at 128 x 128 x 32 x 32 with 3 x 3 windows).  Batches whose buffers
    // would exceed 256 MiB each are processed in parts of whole samples, grad_weight accumulating
    // over the parts: the scratch stays bounded whatever the batch, at a small cost in time (the parts are long enough
    // to fill the device and grad_weight is added with atomics from the second row chunk on anyway: three parts of
    // 43 samples at that shape take 4 % longer than one piece).
    // Where the kernel gathers, the one buffer may be twice as large: the same 512 MiB in all, in fewer parts.
    size_t budget = 256u << 20;
    if (const char* mb = getenv("NORM_DIST_CONV_PART_MB")) {  // tuning / test aid: budget per buffer in MiB
        if (atof(mb) > 0) budget = (size_t)(atof(mb) * 1048576.0);
    }
    if (norm_backward_gathers(s, p)) budget *= 2;
    const size_t per_sample = (size_t)s.CIg * s.G * s.HW * sizeof(float);
    int part = (int)std::max<size_t>(1, budget / std::max<size_t>(1, per_sample));
    part = ceil_div(B, ceil_div(B, part));  // parts of equal size
    if (B <= part)
        return launch_norm_backward(grad_output, input, weight, output, s, grad_input, grad_weight, p,
                                    (hipStream_t)stream, &u);
    if (grad_weight != nullptr) {
        if (int rc = fill_zero(grad_weight, (long)s.COg * s.G * s.CIg, (hipStream_t)stream)) return rc;
    }
    const long out_stride = (long)CO * s.HW, img_stride = (long)C * H * W;
    for (int b0 = 0; b0 < B; b0 += part) {
        const int nb = std::min(part, B - b0);
        UnfoldGeom up;
        Geom sp;
        if (int rc = make_conv_geom(nb, C, H, W, CO, G, kernel_h, kernel_w, dilation_h, dilation_w, padding_h, padding_w,
                                    stride_h, stride_w, &up, &sp))
            return rc;
        if (int rc = launch_norm_backward(grad_output + b0 * out_stride, input + b0 * img_stride, weight,
                                          output + b0 * out_stride, sp, grad_input + b0 * img_stride, grad_weight, p,
                                          (hipStream_t)stream, &up, grad_weight != nullptr))
            return rc;
    }
    return NDIST_OK;
}

int ndist_conv_norm_dist_backward_input(const float* grad_output, const float* input, const float* weight,
                                        const float* output, int B, int C, int H, int W, int CO, int G, int kernel_h,
                                        int kernel_w, int dilation_h, int dilation_w, int padding_h, int padding_w,
                                        int stride_h, int stride_w, float* grad_input, float p, ndist_stream_t stream) {
    return conv_norm_backward(grad_output, input, weight, output, B, C, H, W, CO, G, kernel_h, kernel_w, dilation_h,
                              dilation_w, padding_h, padding_w, stride_h, stride_w, grad_input, nullptr, p, stream);
}

int ndist_conv_norm_dist_backward_input_weight(const float* grad_output, const float* input, const float* weight,
                                               const float* output, int B, int C, int H, int W, int CO, int G,
                                               int kernel_h, int kernel_w, int dilation_h, int dilation_w, int padding_h,
                                               int padding_w, int stride_h, int stride_w, float* grad_input,
                                               float* grad_weight, float p, ndist_stream_t stream) {
    NDIST_REQUIRE(grad_weight);
    return conv_norm_backward(grad_output, input, weight, output, B, C, H, W, CO, G, kernel_h, kernel_w, dilation_h,
                              dilation_w, padding_h, padding_w, stride_h, stride_w, grad_input, grad_weight, p, stream);
}

static int conv_backward(const float* g1, const float* g2, const int32_t* p1, const int32_t* p2, const UnfoldGeom& u,
                         const Geom& s, float* gx1, float* gx2, float* gw, hipStream_t st) {
    const bool bound = g2 != nullptr;
    int rc = bound ? launch_bound_backward(g1, g2, p1, p2, s, gx1, gx2, gw, st, &u)
                   : launch_inf_backward(g1, p1, s, gx1, gw, st, &u);
    if (rc != -1) return rc;
    const size_t n = (size_t)s.M * s.CIg * s.G;
    float* scratch = nullptr;
    NDIST_HIP_TRY(scratch_alloc((void**)&scratch, (bound ? 2 : 1) * n * sizeof(float), st));
    rc = bound ? launch_bound_backward(g1, g2, p1, p2, s, scratch, scratch + n, gw, st)
               : launch_inf_backward(g1, p1, s, scratch, gw, st);
    if (!rc) rc = launch_fold(scratch, u, gx1, st);
    if (!rc && bound) rc = launch_fold(scratch + n, u, gx2, st);
    if (hip_failed(scratch_free(scratch, st)) && !rc) rc = NDIST_ERR_HIP;
    return rc;
}

int ndist_conv_inf_dist_backward_input(const float* grad_output, const int32_t* pos, int B, int C, int H, int W, int CO,
                                       int G, int kernel_h, int kernel_w, int dilation_h, int dilation_w, int padding_h,
                                       int padding_w, int stride_h, int stride_w, float* grad_input,
                                       ndist_stream_t stream) {
    NDIST_REQUIRE(grad_output); NDIST_REQUIRE(pos); NDIST_REQUIRE(grad_input);
    UnfoldGeom u;
    Geom s;
    if (int rc = make_conv_geom(B, C, H, W, CO, G, kernel_h, kernel_w, dilation_h, dilation_w, padding_h, padding_w,
                                stride_h, stride_w, &u, &s))
        return rc;
    return conv_backward(grad_output, nullptr, pos, nullptr, u, s, grad_input, nullptr, nullptr, (hipStream_t)stream);
}

int ndist_conv_inf_dist_backward_input_weight(const float* grad_output, const int32_t* pos, int B, int C, int H, int W,
                                              int CO, int G, int kernel_h, int kernel_w, int dilation_h, int dilation_w,
                                              int padding_h, int padding_w, int stride_h, int stride_w,
                                              float* grad_input, float* grad_weight, ndist_stream_t stream) {
    NDIST_REQUIRE(grad_output); NDIST_REQUIRE(pos); NDIST_REQUIRE(grad_input); NDIST_REQUIRE(grad_weight);
    UnfoldGeom u;
    Geom s;
    if (int rc = make_conv_geom(B, C, H, W, CO, G, kernel_h, kernel_w, dilation_h, dilation_w, padding_h, padding_w,
                                stride_h, stride_w, &u, &s))
        return rc;
    return conv_backward(grad_output, nullptr, pos, nullptr, u, s, grad_input, nullptr, grad_weight, (hipStream_t)stream);
}

int ndist_conv_bound_inf_dist_backward_input(const float* grad_outputL, const float* grad_outputU, const int32_t* posL,
                                             const int32_t* posU, int B, int C, int H, int W, int CO, int G, int kernel_h,
                                             int kernel_w, int dilation_h, int dilation_w, int padding_h, int padding_w,
                                             int stride_h, int stride_w, float* grad_inputL, float* grad_inputU,
                                             ndist_stream_t stream) {
    NDIST_REQUIRE(grad_outputL); NDIST_REQUIRE(grad_outputU); NDIST_REQUIRE(posL); NDIST_REQUIRE(posU);
    NDIST_REQUIRE(grad_inputL); NDIST_REQUIRE(grad_inputU);
    UnfoldGeom u;
    Geom s;
    if (int rc = make_conv_geom(B, C, H, W, CO, G, kernel_h, kernel_w, dilation_h, dilation_w, padding_h, padding_w,
                                stride_h, stride_w, &u, &s))
        return rc;
    return conv_backward(grad_outputL, grad_outputU, posL, posU, u, s, grad_inputL, grad_inputU, nullptr,
                         (hipStream_t)stream);
}

int ndist_conv_bound_inf_dist_backward_input_weight(const float* grad_outputL, const float* grad_outputU,
                                                    const int32_t* posL, const int32_t* posU, int B, int C, int H, int W,
                                                    int CO, int G, int kernel_h, int kernel_w, int dilation_h,
                                                    int dilation_w, int padding_h, int padding_w, int stride_h,
                                                    int stride_w, float* grad_inputL, float* grad_inputU,
                                                    float* grad_weight, ndist_stream_t stream) {
    NDIST_REQUIRE(grad_outputL); NDIST_REQUIRE(grad_outputU); NDIST_REQUIRE(posL); NDIST_REQUIRE(posU);
    NDIST_REQUIRE(grad_inputL); NDIST_REQUIRE(grad_inputU); NDIST_REQUIRE(grad_weight);
    UnfoldGeom u;
    Geom s;
    if (int rc = make_conv_geom(B, C, H, W, CO, G, kernel_h, kernel_w, dilation_h, dilation_w, padding_h, padding_w,
                                stride_h, stride_w, &u, &s))
        return rc;
    return conv_backward(grad_outputL, grad_outputU, posL, posU, u, s, grad_inputL, grad_inputU, grad_weight,
                         (hipStream_t)stream);
}

}  // extern "C"
