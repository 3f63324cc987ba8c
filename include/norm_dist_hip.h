/*
 * C ABI of the MI355X (gfx950) L_p-distance operator library, libnorm_dist_hip.so.
 *
 * One entry point per static member function of the reference's kernel interface
 * (core/cuda/norm_dist.h:4-38 in the reference checkout), with the same argument order and meaning.
 * Differences, all additive:
 *   - every function returns an int status (0 = success, see ndist_status) instead of void;
 *   - every function takes the HIP stream to launch on as its last argument (NULL = the default stream);
 *     the reference always launches on the legacy default stream;
 *   - the integer template parameter `ip` of norm_dist<ip> is chosen inside the library from `p`
 *     (the reference does this in core/cuda/norm_dist.cpp:14-35).
 *
 * Conventions (core/cuda/norm_dist_cuda.cu:72,84,143):
 *   all pointers are DEVICE pointers to contiguous fp32 / int32 arrays on the current HIP device;
 *   input   [B, CI, HW]        CI = G * CI_per_group
 *   weight  [CO, CI / G]       CO = G * CO_per_group
 *   output  [B, CO, HW]
 *   pos     int32 [B, CO, HW]  low 31 bits: arg-max index inside the group, bit 31: sign flag
 *   B, CO, CI, G, HW are the FULL sizes (not per group), as in the reference.
 * The caller allocates every output; the library writes each output element exactly once (gradients are fully
 * overwritten: the caller does not need to zero them).  Calls are asynchronous with respect to the host and
 * ordered on `stream`.  Temporary device memory, where a kernel needs it, comes from arenas the library keeps per
 * (device, stream) and hands to one call at a time (see ndist_release_scratch); nothing else is kept between
 * calls, and the library is re-entrant from several host threads.
 */
#ifndef NORM_DIST_HIP_H
#define NORM_DIST_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef void* ndist_stream_t; /* a hipStream_t */

enum ndist_status {
    NDIST_OK = 0,
    NDIST_ERR_NULL_POINTER = 1,   /* a required pointer is NULL */
    NDIST_ERR_BAD_SHAPE = 2,      /* non-positive size, CI or CO not divisible by G, or a size product overflowing int32 */
    NDIST_ERR_BAD_P = 3,          /* p <= 0, NaN, or infinite where a finite p is required */
    NDIST_ERR_HIP = 4,            /* a HIP runtime call failed; see ndist_last_hip_error() */
    NDIST_ERR_NO_DEVICE = 5,      /* no HIP device is usable */
    NDIST_ERR_CAPTURE = 6,        /* the stream is being captured into a HIP graph and the call needs temporary device
                                     memory from the library's arenas: nothing was allocated or launched */
    NDIST_ERR_TOO_LARGE = 7       /* ndist_*_noalloc: the problem needs more scratch than the fixed array holds */
};

/* Library version (major * 10000 + minor * 100 + patch). */
int ndist_version(void);
/* Human-readable text for a status code. */
const char* ndist_status_string(int status);
/* hipError_t value of the most recent failing HIP call on the calling thread (0 if none). */
int ndist_last_hip_error(void);

/* Measurement aid with no counterpart in the reference: while enabled, every entry point brackets its dominant
 * kernel (the tiled forward kernel, the fused backward kernel, the scatter kernel) with two HIP events on the launch
 * stream.  ndist_last_kernel_ms() waits for the most recent such kernel launched by any thread of the process and
 * returns its duration (one profiled caller at a time); status NDIST_ERR_BAD_SHAPE means nothing has been recorded. */
void ndist_set_profiling(int enable);
int ndist_last_kernel_ms(float* ms);
/* Tuning and test aid, no counterpart in the reference.  For exponents p >= 16 on large problems the library queues
 * several variants of its kernels and lets device-side probes of the data choose one.  skip: -1 the probes decide
 * (default), 0 never, 1 always run the pair-skipping variants (forced on, also for small problems); bounds: the same
 * for the choice between the two skipping variants of the backward.  skip also governs the k-tile skipping of
 * the p = inf and interval-bound forwards (on by default for large fully-connected problems).  The setting belongs to the
 * calling host thread (it governs the entry points that thread calls afterwards; other threads are unaffected); -1
 * returns to the value the environment gave when the library was loaded: NORM_DIST_SKIP, NORM_DIST_BWD_BOUNDS = 0 / 1.  Results agree within the operator's tolerance
 * whichever variant runs. */
void ndist_set_skip_mode(int skip, int bounds);
/* Tuning and test aid, no counterpart in the reference.  On the problems whose p = inf forward skips k-tiles the
 * library first finds out on the device whether a few 32-wide k-tiles per row of x, or per row of w, decide every
 * maximum (activations with a few outliers against small weights; weights with one large planted entry per row) and
 * then computes the outputs from those tiles alone; results are bit-identical either way.  mode: -1 the counts
 * decide (default), 0 never, 1 always the cheaper side, 2 always the rows of x, 3 always the rows of w.
 * Per calling host thread, like ndist_set_skip_mode; -1 returns to the value of NORM_DIST_HOT at load time (or to
 * the default). */
void ndist_set_hot_mode(int mode);
/* Tuning and test aid, no counterpart in the reference.  For 10 < p <= 48 in the fully connected layout the forward
 * normalises the sum by a bound of the maximum known before the reduction starts (largest |x| of the row plus
 * largest |w|) and so needs one pass over the pairs instead of two; outputs whose sum leaves the safe float range
 * under that bound are recomputed with their exact maximum.  mode: -1 for problems of 2e7 pairs and more (default),
 * 0 never, 1 whenever the layout allows.  Per calling host thread; -1 returns to NORM_DIST_ROW_SCALE (or the default).  Results agree within
 * the operator's tolerance either way. */
void ndist_set_scaled_mode(int mode);
/* The calling host thread's current values of the three settings above (null pointers are skipped). */
void ndist_get_modes(int* skip, int* bounds, int* hot, int* scaled);
/* No counterpart in the reference (PyTorch's caching allocator plays this role there).  Entry points that need
 * temporary device memory (finite-p backward, forwards whose k range is split over workgroups, the large-p paths,
 * the conv fallback) take it from arenas the library keeps per (device, stream): allocated with hipMalloc the first
 * time a stream needs that much, then reused by every later call on the stream, which is why those calls neither
 * allocate nor wait for the stream once warmed up.  This call frees the arenas that no running call is using; it
 * waits for the device.  Returns a status code. */
int ndist_release_scratch(void);
/* Test aid, no counterpart in the reference: hipMalloc / hipFree calls the library has made for its arenas since it
 * was loaded (either pointer may be NULL).  Unchanged across a call = that call allocated nothing. */
void ndist_scratch_counters(long* mallocs, long* frees);
/* HIP graphs: an entry point that would take arena scratch returns NDIST_ERR_CAPTURE when `stream` is being captured
 * (before it allocates or launches anything): a captured graph must not hold addresses of memory a later call may
 * free.  Entry points and shapes that need no scratch can be captured; ndist_norm_dist_backward_input_weight_noalloc
 * never takes arena scratch. */

/* ---- finite p: replaces template struct norm_dist<ip> (core/cuda/norm_dist.h:4-14) ------------------- */

/* norm_dist<ip>::forward_with_max(max_output = nullptr) for p <= 10 and norm_dist<ip>::forward for p > 10, chosen
 * as core/cuda/norm_dist.cpp:40-53 does: output = ||input - weight||_p over the CI/G axis. */
int ndist_norm_dist_forward(const float* input, const float* weight,
                            int B, int CO, int CI, int G, int HW, float* output, float p, ndist_stream_t stream);

/* norm_dist<ip>::forward_with_max with a caller-supplied normaliser (core/cuda/norm_dist.cpp:55-64):
 * output = max_output * (sum (|input - weight| / max_output)^p + (1e-10 / max_output)^p)^(1/p). */
int ndist_norm_dist_forward_with_max(const float* input, const float* weight, const float* max_output,
                                     int B, int CO, int CI, int G, int HW, float* output, float p,
                                     ndist_stream_t stream);

/* norm_dist<ip>::backward_input (core/cuda/norm_dist.cpp:66-77): grad_input only. `output` is the forward result. */
int ndist_norm_dist_backward_input(const float* grad_output, const float* input, const float* weight,
                                   const float* output, int B, int CO, int CI, int G, int HW,
                                   float* grad_input, float p, ndist_stream_t stream);

/* norm_dist<ip>::backward_input_weight (core/cuda/norm_dist.cpp:79-91): grad_input and grad_weight in one pass. */
int ndist_norm_dist_backward_input_weight(const float* grad_output, const float* input, const float* weight,
                                          const float* output, int B, int CO, int CI, int G, int HW,
                                          float* grad_input, float* grad_weight, float p, ndist_stream_t stream);

/* No counterpart in the reference.  For callers that cannot allocate device memory at the time of the call (code
 * under HIP graph capture, serving loops and harnesses that forbid hipMalloc): the same computation and arguments as
 * ndist_norm_dist_backward_input_weight, but every byte of temporary device memory (the per-(row, output) factor
 * array of the fused kernel, and the few words of the large-exponent probes) comes from one fixed array of
 * ndist_noalloc_scratch_bytes() = 24 MiB that is part of the library's code object and that every GPU holds until
 * the process ends.  The call makes no hipMalloc / hipFree / event creation, whatever the arenas hold.  Problems whose factor
 * array, G*CO/G x (B*HW rounded up to the kernel's row chunk) floats (twice that for 1 < p < 2), exceeds the array
 * return NDIST_ERR_TOO_LARGE before anything is launched (B*HW x CO up to 6.29 M, e.g. 512 x 5120 twice over); the
 * conv layout runs without the transposed copies of the allocating entry point when they do not fit.  All calls on
 * one GPU share that GPU's array: calls that overlap in time on one device (two streams, two threads) race; calls
 * queued on one stream do not.  Results are those of ndist_norm_dist_backward_input_weight.
 * Under graph capture: the array's device address and the device's properties are looked up once per device, by
 * ndist_noalloc_prepare() or by the first call made outside a capture; a call on a capturing stream that finds
 * them missing returns NDIST_ERR_CAPTURE and launches nothing.  A graph that holds such a call also holds the
 * array's address: replays race with any other use of the array on that GPU that overlaps them in time. */
int ndist_noalloc_prepare(void); /* once per device, that device current, outside any capture; no counterpart either */
int ndist_norm_dist_backward_input_weight_noalloc(const float* grad_output, const float* input, const float* weight,
                                                  const float* output, int B, int CO, int CI, int G, int HW,
                                                  float* grad_input, float* grad_weight, float p,
                                                  ndist_stream_t stream);
size_t ndist_noalloc_scratch_bytes(void);

/* ---- p = infinity: replaces struct inf_dist (core/cuda/norm_dist.h:16-25) ---------------------------- */

/* inf_dist::forward_nograd: output = max(1e-10, max_ci |input - weight|). */
int ndist_inf_dist_forward_nograd(const float* input, const float* weight,
                                  int B, int CO, int CI, int G, int HW, float* output, ndist_stream_t stream);

/* inf_dist::forward: same value plus pos = first index attaining it (lowest index wins ties), bit 31 set when
 * input - weight < 0 there; pos = 0 when nothing exceeds 1e-10. */
int ndist_inf_dist_forward(const float* input, const float* weight,
                           int B, int CO, int CI, int G, int HW, float* output, int32_t* pos, ndist_stream_t stream);

/* inf_dist::backward_input: grad_input[b, idx, hw] = sum over co of +-grad_output routed by pos. */
int ndist_inf_dist_backward_input(const float* grad_output, const int32_t* pos,
                                  int B, int CO, int CI, int G, int HW, float* grad_input, ndist_stream_t stream);

/* inf_dist::backward_input_weight: additionally grad_weight[co, idx] = -sum over (b, hw) of the same values. */
int ndist_inf_dist_backward_input_weight(const float* grad_output, const int32_t* pos,
                                         int B, int CO, int CI, int G, int HW,
                                         float* grad_input, float* grad_weight, ndist_stream_t stream);

/* ---- interval bounds of the infinity distance: replaces struct bound_inf_dist (core/cuda/norm_dist.h:27-38) */

int ndist_bound_inf_dist_forward_nograd(const float* inputL, const float* inputU, const float* weight,
                                        int B, int CO, int CI, int G, int HW,
                                        float* outputL, float* outputU, ndist_stream_t stream);

int ndist_bound_inf_dist_forward(const float* inputL, const float* inputU, const float* weight,
                                 int B, int CO, int CI, int G, int HW,
                                 float* outputL, float* outputU, int32_t* posL, int32_t* posU,
                                 ndist_stream_t stream);

int ndist_bound_inf_dist_backward_input(const float* grad_outputL, const float* grad_outputU,
                                        const int32_t* posL, const int32_t* posU,
                                        int B, int CO, int CI, int G, int HW,
                                        float* grad_inputL, float* grad_inputU, ndist_stream_t stream);

int ndist_bound_inf_dist_backward_input_weight(const float* grad_outputL, const float* grad_outputU,
                                               const int32_t* posL, const int32_t* posU,
                                               int B, int CO, int CI, int G, int HW,
                                               float* grad_inputL, float* grad_inputU, float* grad_weight,
                                               ndist_stream_t stream);

/* ---- a layer's distance and its interval bounds in one call ---------------------------------------------------
 * No counterpart in the reference's kernel interface: its layers call inf_dist::forward[_nograd] and
 * bound_inf_dist::forward[_nograd] one after the other on the same weights (core/modules/norm_dist.py:30-34), which is
 * what certification does on every layer.  These entry points compute exactly what those two calls compute (same
 * values, same codes) and share the pre-pass over the weights between them where the k-tile skipping variants run. */
int ndist_inf_and_bound_forward_nograd(const float* input, const float* inputL, const float* inputU, const float* weight,
                                       int B, int CO, int CI, int G, int HW, float* output, float* outputL,
                                       float* outputU, ndist_stream_t stream);
int ndist_inf_and_bound_forward(const float* input, const float* inputL, const float* inputU, const float* weight, int B,
                                int CO, int CI, int G, int HW, float* output, int32_t* pos, float* outputL,
                                float* outputU, int32_t* posL, int32_t* posU, ndist_stream_t stream);

/* ---- evaluation with the weights' pre-pass kept between calls ---------------------------------------------------
 * No counterpart in the reference.  On large fully connected problems the p = inf forwards start with a pass over the
 * weights (largest magnitude, its position and the 32-wide tile maxima of every row: it reads all of w).  While the
 * weights do not change -- evaluation, certification, serving -- that pass can be done once:
 *   ndist_weight_cache_bytes      size of the caller-allocated device buffer for a [CO, CI / G] weight (0: bad shape)
 *   ndist_weight_cache_prepare    fills it from `weight` (one kernel)
 *   ..._nograd_cached             ndist_inf_dist_forward_nograd / ndist_inf_and_bound_forward_nograd reading the pass
 *                                 from `cache` instead of redoing it; results are bit-identical.
 * The cache is only valid for the weight values it was prepared from: prepare it again after every change of the
 * weights (the library cannot check).  Problems that use no pre-pass (small ones, the conv layout) ignore it. */
long long ndist_weight_cache_bytes(int CO, int CI, int G);
int ndist_weight_cache_prepare(const float* weight, int CO, int CI, int G, void* cache, ndist_stream_t stream);
int ndist_inf_dist_forward_nograd_cached(const float* input, const float* weight, const void* cache, int B, int CO, int CI,
                                         int G, int HW, float* output, ndist_stream_t stream);
int ndist_inf_and_bound_forward_nograd_cached(const float* input, const float* inputL, const float* inputU,
                                              const float* weight, const void* cache, int B, int CO, int CI, int G, int HW,
                                              float* output, float* outputL, float* outputU, ndist_stream_t stream);

/* ---- mean shift and bias of a distance layer ------------------------------------------------------------------
 * The reference has no kernel of its own here: every layer follows the operator with MeanShift and a bias add
 * written in torch primitives (core/modules/norm_dist.py:35-38, core/modules/basic_modules.py:121-132).  These two
 * entry points do the same in one launch (fully connected layout, C % 4 == 0) or two to three.  Tensors are [B, C, HW] like the operator's outputs.
 *   forward:  mean[c] = training ? mean over (b, hw) of x : running_mean[c]   (0 when running_mean is NULL in evaluation)
 *             y* = t* - mean[c] + bias1[c] + bias2[c]     for t* in {x, lower, upper} that are not NULL
 *             training also writes mean_out[c] = mean[c] and running_mean[c] = (1 - momentum) running_mean[c] + momentum mean[c]
 *             (running_mean may be NULL in training; bias1, bias2 may be NULL; x is required in training)
 *   backward: colsum_out[c] = sum over (b, hw) of the given gradients (the gradient of either bias; may be NULL);
 *             training: grad_x = grad_y - colsum / (B HW)  (grad_y required then; mean_scratch: [C] floats of the
 *             caller's);  evaluation: grad_x is grad_y itself and is not written.
 *             The gradients of lower and upper pass through unchanged and are not touched.
 * Sums are taken in a fixed order: results repeat bit for bit. */
int ndist_mean_shift_forward(const float* x, const float* lower, const float* upper, int B, int C, int HW, int training,
                             float momentum, float* running_mean, const float* bias1, const float* bias2,
                             float* mean_out, float* y, float* y_lower, float* y_upper, ndist_stream_t stream);
int ndist_mean_shift_backward(const float* grad_y, const float* grad_y_lower, const float* grad_y_upper, int B, int C,
                              int HW, int training, float* grad_x, float* colsum_out, float* mean_scratch,
                              ndist_stream_t stream);

/* Tail of a distance network, no kernels of their own in the reference either (ell_inf_models.py:41-46 and
 * main.py:304-310 in torch primitives): the worst-case margins
 *   margin[b, c] = (upper[b, t_b] - lower[b, c]) / (2 eps) for c != t_b, 0 for c == t_b        (t = targets, int64)
 * of the logits -x (lower / upper NULL: x - eps / x + eps, the network being 1-Lipschitz in the infinity norm), and
 * the hinge loss on them, loss = (1 - mix) * mean_b max_c relu(margin) + mix * mean relu(margin).  All tensors
 * [B, C] contiguous; argmax [B] int32 links ndist_hinge_forward to its backward; loss and grad_loss are one float on
 * the device.  The backward entry points overwrite their outputs (grad_x, or grad_lower and grad_upper; pass NULL
 * for those that do not exist).  Sums in a fixed order. */
int ndist_margin_forward(const float* x, const float* lower, const float* upper, const long long* targets, int B, int C,
                         float eps, float* margin, ndist_stream_t stream);
int ndist_margin_backward(const float* grad_margin, const long long* targets, int B, int C, float eps, float* grad_x,
                          float* grad_lower, float* grad_upper, ndist_stream_t stream);
int ndist_hinge_forward(const float* margin, int B, int C, float mix, float* loss, int* argmax, ndist_stream_t stream);
int ndist_hinge_backward(const float* margin, const int* argmax, const float* grad_loss, int B, int C, float mix,
                         float* grad_margin, ndist_stream_t stream);

/* ---- patch extraction for the convolutional layer -------------------------------------------------------------
 * The reference has no kernel of its own here: NormDistConv calls torch.nn.functional.unfold
 * (core/modules/norm_dist.py:93-102).  These two entry points replace that call and its autograd adjoint with one
 * launch per batch; sizes and semantics are those of torch.nn.functional.unfold / fold.
 *   input        [B, C, H, W]
 *   output       [B, C * kernel_h * kernel_w, OH * OW],  OH = (H + 2*padding_h - dilation_h*(kernel_h-1) - 1) / stride_h + 1
 *   grad_output  like output;  grad_input like input (fully overwritten) */
int ndist_unfold_forward(const float* input, int B, int C, int H, int W, int kernel_h, int kernel_w, int dilation_h,
                         int dilation_w, int padding_h, int padding_w, int stride_h, int stride_w, float* output,
                         ndist_stream_t stream);
int ndist_unfold_backward(const float* grad_output, int B, int C, int H, int W, int kernel_h, int kernel_w,
                          int dilation_h, int dilation_w, int padding_h, int padding_w, int stride_h, int stride_w,
                          float* grad_input, ndist_stream_t stream);

/* ---- convolutional layer without the unfolded tensor ------------------------------------------------------------
 * NormDistConv.forward (core/modules/norm_dist.py:93-102) unfolds x (and both bounds) to [B, C*kh*kw, OH*OW] and calls
 * the operators above; these entry points take the images themselves and extract the patches while the kernel
 * loads its tiles.  Results are bit-identical to ndist_unfold_forward followed by the corresponding entry point
 * (inf_dist / bound_inf_dist forward, forward_nograd, core/cuda/norm_dist.h:14-38), values and arg-max codes alike;
 * the backward entry points produce the image gradients directly, i.e. the corresponding backward followed by
 * ndist_unfold_backward, without the unfolded gradient ever being written (geometries whose image plane does not
 * fit the kernels' LDS budget fall back to exactly that sequence in scratch memory).
 *   input(L,U), grad_input(L,U)  [B, C, H, W]      weight, grad_weight  [CO, C / G * kernel_h * kernel_w]
 *   output(L,U), pos(L,U), grad_output(L,U)  [B, CO, OH * OW]      geometry arguments as for ndist_unfold_forward
 * grad_input(L,U) and grad_weight are fully overwritten. */
int ndist_conv_inf_dist_forward_nograd(const float* input, const float* weight, int B, int C, int H, int W, int CO, int G,
                                       int kernel_h, int kernel_w, int dilation_h, int dilation_w, int padding_h,
                                       int padding_w, int stride_h, int stride_w, float* output, ndist_stream_t stream);
int ndist_conv_bound_inf_dist_forward_nograd(const float* inputL, const float* inputU, const float* weight, int B, int C,
                                             int H, int W, int CO, int G, int kernel_h, int kernel_w, int dilation_h,
                                             int dilation_w, int padding_h, int padding_w, int stride_h, int stride_w,
                                             float* outputL, float* outputU, ndist_stream_t stream);
int ndist_conv_inf_dist_forward(const float* input, const float* weight, int B, int C, int H, int W, int CO, int G,
                                int kernel_h, int kernel_w, int dilation_h, int dilation_w, int padding_h, int padding_w,
                                int stride_h, int stride_w, float* output, int32_t* pos, ndist_stream_t stream);
int ndist_conv_bound_inf_dist_forward(const float* inputL, const float* inputU, const float* weight, int B, int C, int H,
                                      int W, int CO, int G, int kernel_h, int kernel_w, int dilation_h, int dilation_w,
                                      int padding_h, int padding_w, int stride_h, int stride_w, float* outputL,
                                      float* outputU, int32_t* posL, int32_t* posU, ndist_stream_t stream);
int ndist_conv_inf_dist_backward_input(const float* grad_output, const int32_t* pos, int B, int C, int H, int W, int CO,
                                       int G, int kernel_h, int kernel_w, int dilation_h, int dilation_w, int padding_h,
                                       int padding_w, int stride_h, int stride_w, float* grad_input,
                                       ndist_stream_t stream);
int ndist_conv_inf_dist_backward_input_weight(const float* grad_output, const int32_t* pos, int B, int C, int H, int W,
                                              int CO, int G, int kernel_h, int kernel_w, int dilation_h, int dilation_w,
                                              int padding_h, int padding_w, int stride_h, int stride_w,
                                              float* grad_input, float* grad_weight, ndist_stream_t stream);
int ndist_conv_bound_inf_dist_backward_input(const float* grad_outputL, const float* grad_outputU, const int32_t* posL,
                                             const int32_t* posU, int B, int C, int H, int W, int CO, int G, int kernel_h,
                                             int kernel_w, int dilation_h, int dilation_w, int padding_h, int padding_w,
                                             int stride_h, int stride_w, float* grad_inputL, float* grad_inputU,
                                             ndist_stream_t stream);
int ndist_conv_bound_inf_dist_backward_input_weight(const float* grad_outputL, const float* grad_outputU,
                                                    const int32_t* posL, const int32_t* posU, int B, int C, int H, int W,
                                                    int CO, int G, int kernel_h, int kernel_w, int dilation_h,
                                                    int dilation_w, int padding_h, int padding_w, int stride_h,
                                                    int stride_w, float* grad_inputL, float* grad_inputU,
                                                    float* grad_weight, ndist_stream_t stream);

/* The finite-p distance on images, same conventions: norm_dist on the patches of `input` (what the reference's
 * NormDistConv computes through torch.nn.functional.unfold + norm_dist::forward / backward_input[_weight],
 * core/modules/norm_dist.py:93-102, core/cuda/norm_dist.h:4-17), without the unfolded tensor: the forward extracts
 * the patches while it loads its tiles; the backward writes them once in the row layout its kernel reads and folds
 * the gradient rows back into the image (scratch: 8 * B * C*kh*kw * OH*OW bytes from the stream's arena).
 *   output, grad_output  [B, CO, OH * OW]    grad_input  [B, C, H, W]    grad_weight  [CO, C/G * kh * kw] */
int ndist_conv_norm_dist_forward(const float* input, const float* weight, int B, int C, int H, int W, int CO, int G,
                                 int kernel_h, int kernel_w, int dilation_h, int dilation_w, int padding_h, int padding_w,
                                 int stride_h, int stride_w, float* output, float p, ndist_stream_t stream);
int ndist_conv_norm_dist_backward_input(const float* grad_output, const float* input, const float* weight,
                                        const float* output, int B, int C, int H, int W, int CO, int G, int kernel_h,
                                        int kernel_w, int dilation_h, int dilation_w, int padding_h, int padding_w,
                                        int stride_h, int stride_w, float* grad_input, float p, ndist_stream_t stream);
int ndist_conv_norm_dist_backward_input_weight(const float* grad_output, const float* input, const float* weight,
                                               const float* output, int B, int C, int H, int W, int CO, int G,
                                               int kernel_h, int kernel_w, int dilation_h, int dilation_w, int padding_h,
                                               int padding_w, int stride_h, int stride_w, float* grad_input,
                                               float* grad_weight, float p, ndist_stream_t stream);

#ifdef __cplusplus
}
#endif
#endif /* NORM_DIST_HIP_H */
