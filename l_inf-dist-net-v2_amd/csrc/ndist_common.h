// Shared declarations of the gfx950 L_p-distance kernels: constants, problem descriptors, host-side helpers.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace ndist {

// Floors and sentinels of the operator (reference: core/cuda/inf_dist_cuda.cu:11,
// core/cuda/bound_inf_dist_cuda.cu:11-12, core/cuda/norm_dist_cuda.cu:13-15).
constexpr float kEps = 1e-10f;
constexpr float kFltMin = 1.175494351e-38f;
constexpr uint32_t kSignBit = 0x80000000u;
constexpr uint32_t kNoGradId = 0xffffffffu;
// Largest p served by the plain (un-normalised) sum; above it the online-max-normalised sum is used
// (reference: core/cuda/norm_dist.cpp:4,44).
constexpr float kMinNormalizedP = 10.0f;

constexpr int kWave = 64;

// Problem geometry shared by every kernel. Sizes are per group unless stated.
struct Geom {
    int B, HW, M;   // M = B * HW rows of the distance "matrix"
    int COg, CIg, G;
    __host__ __device__ int CO() const { return COg * G; }
    __host__ __device__ int CI() const { return CIg * G; }
};

// element offsets in the three tensor layouts
__host__ __device__ inline long x_off(const Geom& s, int b, int g, int ci, int hw) {
    return (((long)b * s.G + g) * s.CIg + ci) * s.HW + hw;
}
__host__ __device__ inline long w_off(const Geom& s, int g, int co, int ci) {
    return ((long)g * s.COg + co) * s.CIg + ci;
}
__host__ __device__ inline long y_off(const Geom& s, int b, int g, int co, int hw) {
    return (((long)b * s.G + g) * s.COg + co) * s.HW + hw;
}

// hardware transcendentals (v_exp_f32 / v_log_f32): base-2, about 1 ulp, no denormal handling
__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }
__device__ __forceinline__ float fast_log2(float x) { return __builtin_amdgcn_logf(x); }

constexpr int ceil_div(int a, int b) { return (a + b - 1) / b; }
constexpr int round_up(int a, int b) { return ceil_div(a, b) * b; }

// host side -----------------------------------------------------------------------------------------------
struct DeviceInfo {
    int num_cu;
    int lds_bytes;
};
// Properties of the current device, queried once per device and cached.
const DeviceInfo& device_info();
bool device_info_cached();  // the current device's properties have been queried already

// Records a failing HIP call for ndist_last_hip_error(); returns true when `e` is an error.
bool hip_failed(hipError_t e);
// The same, as an ndist_status value: 0 for success, NDIST_ERR_CAPTURE when scratch was refused because the stream
// is being captured, NDIST_ERR_TOO_LARGE when the fixed scratch array is too small, else NDIST_ERR_HIP.
int hip_status(hipError_t e);

// Optional timing of the dominant kernel of an entry point (see ndist_set_profiling): when enabled, the launcher
// brackets that one kernel with two events on the launch stream; ndist_last_kernel_ms() reads them back.
struct KernelTimer {
    explicit KernelTimer(hipStream_t st);
    ~KernelTimer();
    hipStream_t stream;
    bool active;
};

// Temporary device memory for the duration of one call, from an arena that the library keeps per (device, stream):
// same shape as hipMallocAsync / hipFreeAsync, but without their wait for the stream's queued work, and without any
// allocation once the arena has grown to the largest request of its stream.  Releases go in reverse order of the
// requests; every request of a call must be released before the call returns.
// A request made while `st` is being captured into a graph fails with hipErrorStreamCaptureUnsupported before
// anything is allocated or launched.
hipError_t scratch_alloc(void** out, size_t bytes, hipStream_t st);
hipError_t scratch_free(void* p, hipStream_t st);
// Frees the memory of every arena no call is using (waits for the device).
int scratch_release_all();
// hipMalloc / hipFree calls made on behalf of the arenas since the library was loaded
void scratch_counters(long* mallocs, long* frees);
// true while `st` is being captured into a graph (or its state cannot be queried)
bool stream_is_capturing(hipStream_t st);

// Scratch without any allocation: a fixed array of kStaticScratchBytes in device memory, one copy per device.  While
// a StaticScratchScope lives on the calling thread, scratch_alloc serves from that array (stack-ordered, failing
// with hipErrorOutOfMemory beyond its size) and calls no allocator; calls that overlap on one device share the
// array and race.
constexpr size_t kStaticScratchBytes = 24u << 20;
struct StaticScratchScope {
    explicit StaticScratchScope(bool may_query = true);  // false: never look the array's address up (capture)
    ~StaticScratchScope();
    StaticScratchScope(const StaticScratchScope&) = delete;
    StaticScratchScope& operator=(const StaticScratchScope&) = delete;
    hipError_t status;  // of the one-time address lookup
    char* base;         // device address of this device's copy of the array
    size_t used;
    int live;
};
bool static_scratch_active();
hipError_t static_scratch_base(char** out, bool may_query);

// Seeds and k-tile bounds for the forward operators that skip whole k-tiles (fully-connected layout, HW == 1).
//   seed    [M][COg*G] as the output: for every output, the larger of the two pairs |x - w| at the k where its x row
//           and where its w row is largest in magnitude (a lower bound of the output's maximum, an actual pair)
//   tile_x  [rows of x][ntile], tile_w [rows of w][ntile]: the largest magnitude inside every 32-wide k-tile
// `base` points at seed_scratch_floats(s) floats of scratch (twice that for the interval bounds); with a gate the
// kernels do nothing unless gate[0] < gate_limit.
// Interval bounds (x = lower, x2 = upper input bound): tile_x covers both arrays, and the seeds are the pairs
// max(w - xL, xU - w) / min(w - xL, xU - w) at the same two k.
// The pre-passes read all of w once: they pay from about this many rows of x on (measured at 5120 x 5120).
constexpr int kMinSeededRows = 192;
struct SeedBuffers {
    float* seed;
    float* seed2;  // interval bounds only (x2 != nullptr): seed of the lower reduction, `seed` that of the upper one
    float* tile_x;
    float* tile_w;
    int ntile;
    // per row of x / of w: the element of largest magnitude (NaN when the row holds a NaN) and its k
    float* seed_x;
    int32_t* seed_k;
    float* seed_w;
    int32_t* seed_wk;
    // interval bounds only: per row of the box the largest max(-lower, upper) and max(lower, -upper) over k
    float* far_hi;
    float* far_lo;
};
// The part of the pre-passes that depends on w alone (per row of w: largest element, its k, tile maxima): two
// operators called on the same weights (a layer's distance and its interval bounds) can share it.
struct WeightSeeds {
    float* seed_w;
    int32_t* seed_wk;
    float* tile_w;
};
size_t seed_scratch_floats(const Geom& s);
size_t bound_seed_scratch_floats(const Geom& s);  // with the second seed array and the row statistics of the box
size_t weight_seed_floats(const Geom& s);
WeightSeeds weight_seeds_at(float* base, const Geom& s);  // the three arrays inside weight_seed_floats(s) floats
int launch_weight_seeds(const float* w, const Geom& s, float* base, const int* gate, int gate_limit, hipStream_t st,
                        WeightSeeds* out);
// `wpre`: weight rows already done by launch_weight_seeds (their part of `base` then stays unused)
int launch_seeds(const float* x, const float* w, const Geom& s, float* base, const int* gate, int gate_limit,
                 hipStream_t st, SeedBuffers* out, const float* x2 = nullptr, const WeightSeeds* wpre = nullptr);
// The two steps of launch_seeds: the row kernels (row seeds, tile bounds), then the seed of every output.
// `zero`: four ints the row kernel clears on the way (counters of kernels queued behind it).
int launch_row_seeds(const float* x, const float* w, const Geom& s, float* base, const int* gate, int gate_limit,
                     hipStream_t st, SeedBuffers* out, const float* x2 = nullptr, const WeightSeeds* wpre = nullptr,
                     int* zero = nullptr);
int launch_output_seeds(const float* x, const float* w, const Geom& s, const SeedBuffers& sb, const int* gate,
                        int gate_limit, hipStream_t st, const float* x2 = nullptr);
// The row kernels of a layer's distance (x into `base`) and of its interval bounds (the box xl, xu into `base_box`)
// in one launch, with the rows of w unless `wpre` brings them; `zero`, `zero_box`: as `zero` above, one per operator.
int launch_joint_row_seeds(const float* x, const float* xl, const float* xu, const float* w, const Geom& s, float* base,
                           float* base_box, const WeightSeeds* wpre, hipStream_t st, SeedBuffers* out,
                           SeedBuffers* out_box, int* zero, int* zero_box);
// What the caller of a joint call has queued for one of its two operators before the operator's own launcher runs:
// scratch (owned by the caller), the results of the row pre-pass, and whether the hot-tile plan is among it.
struct SharedFront {
    float* scratch;
    SeedBuffers sb;
    bool plan_done;
};

// p = inf forward through hot k-tiles (fwd_hot.hip).  Queues the kernels that decide, from the row seeds and tile
// bounds in `sb`, whether few enough k-tiles can hold the maxima, and the kernels that then compute out (and pos
// unless null) from those tiles alone.  *decision points at an int that is 0 on the device when they did not run:
// the caller queues the dense kernels gated on it (run while decision[0] < 1).  `base`: hot_scratch_floats(s) floats.
// Mode (ndist_set_hot_mode / NORM_DIST_HOT): -1 the counts decide, 0 off, 1 always the cheaper side, 2 / 3 always the
// rows of x / of w.
// `base` starts with the four ints the row pre-pass has to clear (launch_row_seeds' `zero`).
// with_seeds: when the decision is 0, the last of these launches computes the output seeds in sb.seed (and sb.seed2)
// that launch_output_seeds would: the caller then does not queue that kernel.
// plan_done: the deciding kernel has been queued already (launch_joint_hot_plan, for both operators of a joint call).
bool hot_forward_applies(const Geom& s);
bool hot_alone_applies(const Geom& s);  // fwd_inf.hip: below the size of the seeded kernels, still worth the pre-pass
size_t hot_scratch_floats(const Geom& s);
int launch_inf_hot(const float* x, const float* w, const Geom& s, const SeedBuffers& sb, float* base, float* out,
                   int32_t* pos, hipStream_t st, const int** decision, bool with_seeds, bool plan_done = false);
// the same for the interval bounds (sb from the row pre-pass over both input bounds)
int launch_bound_hot(const float* xl, const float* xu, const float* w, const Geom& s, const SeedBuffers& sb, float* base,
                     float* yl, float* yu, int32_t* pl, int32_t* pu, hipStream_t st, const int** decision,
                     bool with_seeds, bool plan_done = false);
int launch_joint_hot_plan(const Geom& s, const SeedBuffers& sb, float* base, const SeedBuffers& sb_box, float* base_box,
                          hipStream_t st);
void set_hot_mode(int mode);
int hot_mode();

#define NDIST_HIP_TRY(expr)                                        \
    do {                                                           \
        if (int rc_try_ = ::ndist::hip_status((expr))) return rc_try_; \
    } while (0)

// geometry of the patch extraction [B, C, H, W] -> [B, C*kh*kw, OH*OW]
struct UnfoldGeom {
    int B, C, H, W, kh, kw, dh, dw, ph, pw, sh, sw, OH, OW;
};

// Patch extraction as the kernels see it: maps (k, position) of the unfolded problem to an image element, so that a
// kernel can work on images [B, C, H, W] as if they had been unfolded to [B, C*kh*kw, OH*OW] (zeros outside the image).
struct PatchMap {
    int C, H, W, OW, kw, taps, dh, dw, sh, sw, ph, pw, cg;  // taps = kh * kw, cg = image channels per group
    float inv_taps, inv_kw;
    int packable;  // a tap fits one word: channel inside the group below 2^16, pixel offsets below 2^8 each
};
inline PatchMap make_patch_map(const UnfoldGeom& u, int G) {
    const bool packable = u.C / G < (1 << 16) && (u.kh - 1) * (long)u.dh < 256 && (u.kw - 1) * (long)u.dw < 256;
    return PatchMap{u.C, u.H, u.W, u.OW, u.kw, u.kh * u.kw, u.dh, u.dw, u.sh, u.sw, u.ph, u.pw, u.C / G,
                    1.0f / (float)(u.kh * u.kw), 1.0f / (float)u.kw, packable ? 1 : 0};
}

// floor(a / d) for 0 <= a < 2^22 and 0 < d, with inv = 1.0f / d: the float product is off by at most one
__device__ __forceinline__ int small_div(int a, int d, float inv) {
    int q = (int)((float)a * inv);
    const int r = a - q * d;
    q += r >= d ? 1 : 0;
    q -= r < 0 ? 1 : 0;
    return q;
}

// k of group g -> image channel and the tap's pixel offsets inside the window
struct PatchTap {
    int ch, dy, dx;
};
__device__ __forceinline__ PatchTap patch_tap(const PatchMap& c, int g, int k) {
    const int cl = small_div(k, c.taps, c.inv_taps), tap = k - cl * c.taps;
    const int ti = small_div(tap, c.kw, c.inv_kw), tj = tap - ti * c.kw;
    return PatchTap{g * c.cg + cl, ti * c.dh, tj * c.dw};
}
// top-left pixel of the window of output position hw (may lie in the padding)
__device__ __forceinline__ void patch_origin(const PatchMap& c, int hw, int& ih0, int& iw0) {
    const int oh = hw / c.OW, ow = hw - oh * c.OW;
    ih0 = oh * c.sh - c.ph;
    iw0 = ow * c.sw - c.pw;
}
// offset of the image element a tap reads, or -1 when it lies in the padding
__device__ __forceinline__ long patch_offset(const PatchMap& c, int b, const PatchTap& t, int ih0, int iw0) {
    const int ih = ih0 + t.dy, iw = iw0 + t.dx;
    if ((unsigned)ih >= (unsigned)c.H || (unsigned)iw >= (unsigned)c.W) return -1;
    return (((long)b * c.C + t.ch) * c.H + ih) * c.W + iw;
}
__device__ __forceinline__ float patch_elem(const float* __restrict__ x, const PatchMap& c, int b, const PatchTap& t,
                                            int hw) {
    int ih0, iw0;
    patch_origin(c, hw, ih0, iw0);
    const long o = patch_offset(c, b, t, ih0, iw0);
    return o >= 0 ? x[o] : 0.f;
}
// A tap in one word, for tables of taps in LDS (PatchMap::packable): channel << 16 | dy << 8 | dx.
__device__ __forceinline__ int pack_tap(const PatchTap& t) { return (t.ch << 16) | (t.dy << 8) | t.dx; }
__device__ __forceinline__ PatchTap unpack_tap(int v) {
    return PatchTap{(int)((unsigned)v >> 16), (v >> 8) & 0xff, v & 0xff};
}
// four consecutive positions of one output row; (ih0, iw0) is the window origin of the first
__device__ __forceinline__ float4 patch_row4(const float* __restrict__ x, const PatchMap& c, int b, const PatchTap& t,
                                             int ih0, int iw0) {
    float4 r = make_float4(0.f, 0.f, 0.f, 0.f);
    const int ih = ih0 + t.dy, iw = iw0 + t.dx;
    if ((unsigned)ih < (unsigned)c.H) {
        const float* __restrict__ src = x + (((long)b * c.C + t.ch) * c.H + ih) * c.W;
        if ((unsigned)iw < (unsigned)c.W) r.x = src[iw];
        if ((unsigned)(iw + c.sw) < (unsigned)c.W) r.y = src[iw + c.sw];
        if ((unsigned)(iw + 2 * c.sw) < (unsigned)c.W) r.z = src[iw + 2 * c.sw];
        if ((unsigned)(iw + 3 * c.sw) < (unsigned)c.W) r.w = src[iw + 3 * c.sw];
    }
    return r;
}

// kernel launchers (defined one per .hip file); all return an ndist_status value
// device-side probe of the large-p operators: count of sampled pairs above thr * max into gate[0], and the count from
// which the plain (non-skipping) variants are the faster ones
int launch_norm_probe(const float* x, const float* w, const Geom& s, float thr, int* gate, hipStream_t st);
int norm_probe_limit(const Geom& s);
// Tuning and test aid (ndist_set_skip_mode, initial values from NORM_DIST_SKIP / NORM_DIST_BWD_BOUNDS): overrides of the
// device-side probes.  skip: -1 probes decide, 0 never / 1 always use the skipping variants of the large-p kernels
// (forced on, they also serve problems below the size from which they are normally considered); bounds: the same for
// the choice between the two skipping variants of the backward.
int skip_override_limit(int probed_limit);
bool skip_forced_on();
int bounds_override_limit(int probed_limit);
void set_skip_mode(int skip, int bounds);
void get_skip_mode(int* skip, int* bounds);  // the calling thread's current values
// Tuning and test aid (ndist_set_scaled_mode / NORM_DIST_ROW_SCALE): the one-pass normalised forward for
// 10 < p <= 48 in the fully connected layout; -1 from 2e7 pairs on (default), 0 never, 1 whenever the layout allows.
void set_scaled_mode(int mode);
int scaled_mode();
int launch_unfold(const float* x, const UnfoldGeom& u, float* out, hipStream_t st);
int launch_fold(const float* gout, const UnfoldGeom& u, float* gx, hipStream_t st);
// the patches as rows [B * OH * OW][C * kh * kw] (the transpose of the unfolded tensor); -1: geometry not served
int launch_patch_rows(const float* x, const UnfoldGeom& u, float* out, hipStream_t st);
bool patch_rows_applies(const UnfoldGeom& u);
// the adjoint: image gradient from gradient rows [B * OH * OW][C * kh * kw] (any geometry)
int launch_fold_rows(const float* g, const UnfoldGeom& u, float* gx, hipStream_t st);
// The forward launchers take an optional patch geometry `cv`: x (xl, xu) are then images [B, C, H, W], s describes
// the unfolded problem (CIg = C / G * kh * kw, HW = OH * OW) and the kernels extract the patches while loading.
// `front`: the row pre-pass (and the hot-tile plan) of this call are queued already, by launch_inf_bound_forward
int launch_inf_forward(const float* x, const float* w, const Geom& s, float* out, int32_t* pos, hipStream_t st,
                       const UnfoldGeom* cv = nullptr, const WeightSeeds* wpre = nullptr,
                       const SharedFront* front = nullptr);
int launch_bound_forward(const float* xl, const float* xu, const float* w, const Geom& s,
                         float* yl, float* yu, int32_t* pl, int32_t* pu, hipStream_t st,
                         const UnfoldGeom* cv = nullptr, const WeightSeeds* wpre = nullptr,
                         const SharedFront* front = nullptr);
// true when the two launchers above would run their seeded (k-tile skipping) variants on this problem
bool seeded_forward_applies(const Geom& s);
// the distance of x and the interval bounds of (xl, xu) against the same weights, pre-passes over w shared
int launch_inf_bound_forward(const float* x, const float* xl, const float* xu, const float* w, const Geom& s, float* out,
                             int32_t* pos, float* yl, float* yu, int32_t* pl, int32_t* pu, hipStream_t st,
                             const WeightSeeds* cached = nullptr);
int launch_norm_forward(const float* x, const float* w, const float* max_in, const Geom& s, float* out, float p,
                        hipStream_t st);
// on images: s describes the unfolded problem, the kernels extract the patches themselves
int launch_norm_forward_conv(const float* x, const float* w, const Geom& s, float* out, float p, hipStream_t st,
                             const UnfoldGeom& cv);
// With a patch geometry x and gx are images [B, C, H, W] and s describes the unfolded problem: the patches go
// straight into the row layout the kernel reads and the gradient rows are folded back into the image.
// gw_accumulate: grad_weight was zeroed by the caller and is added to (several launches over parts of a batch).
int launch_norm_backward(const float* gout, const float* x, const float* w, const float* out, const Geom& s,
                         float* gx, float* gw, float p, hipStream_t st, const UnfoldGeom* cv = nullptr,
                         bool gw_accumulate = false);
int fill_zero(float* p, long n, hipStream_t st);
// bytes of scratch launch_norm_backward cannot do without (the factor array); everything else it asks for is optional
size_t norm_backward_scratch_bytes(const Geom& s, float p);
// whether the finite-p backward of a conv layer of this (unfolded) geometry gathers its patches from the images, i.e.
// needs one buffer of the unfolded size instead of two
bool norm_backward_gathers(const Geom& s, float p);
// With a patch geometry the input gradients are images [B, C, H, W] (the adjoint of the patch extraction is applied
// on the fly); the launcher returns -1 when the geometry does not fit its kernels and nothing was launched.
int launch_inf_backward(const float* gout, const int32_t* pos, const Geom& s, float* gx, float* gw, hipStream_t st,
                        const UnfoldGeom* cv = nullptr);
int launch_bound_backward(const float* gl, const float* gu, const int32_t* pl, const int32_t* pu, const Geom& s,
                          float* gxl, float* gxu, float* gw, hipStream_t st, const UnfoldGeom* cv = nullptr);

}  // namespace ndist
