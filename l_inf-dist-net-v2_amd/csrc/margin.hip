// Tail of the distance network: worst-case margins and the hinge loss on them, one launch each way instead of
// the two dozen small torch kernels of the reference's formulation (ell_inf_models.py:41-46, main.py:304-310).
//   margins   m[b, c] = (upper[b, t_b] - lower[b, c]) / (2 eps) for c != t_b, 0 for c == t_b
//             (the reference negates the distances first: logits = -x, so the lower bound of a logit is -upper and
//             the margin of class c against the target is ub(logit_c) - lb(logit_t)); without interval bounds the
//             network's Lipschitz property gives lower = x - eps, upper = x + eps
//   hinge     loss = (1 - mix) * mean_b max_c relu(m[b, c]) + mix * mean_{b, c} relu(m[b, c])
// Both are a few thousand elements: one workgroup, sums in a fixed order (reproducible).
#include "../../include/norm_dist_hip.h"
#include "ndist_common.h"

namespace ndist {

__global__ __launch_bounds__(256) void margin_forward_kernel(const float* __restrict__ x, const float* __restrict__ lower,
                                                             const float* __restrict__ upper,
                                                             const long long* __restrict__ targets, int B, int C,
                                                             float eps, float* __restrict__ margin) {
    const long i = (long)blockIdx.x * 256 + threadIdx.x;
    if (i >= (long)B * C) return;
    const int b = (int)(i / C), c = (int)(i - (long)b * C);
    const long long tl = targets[b];
    if (tl < 0 || tl >= C) {  // a label outside the classes must not become a wild read: the row comes out as NaN
        margin[i] = __builtin_nanf("");
        return;
    }
    const int t = (int)tl;
    const float up_t = upper != nullptr ? upper[(long)b * C + t] : x[(long)b * C + t] + eps;
    const float lo_c = lower != nullptr ? lower[i] : x[i] - eps;
    margin[i] = c == t ? 0.f : (up_t - lo_c) / (2.0f * eps);
}

// grad_lower[b, c] = -g[b, c] / (2 eps) (c != t), grad_upper[b, t] = sum_{c != t} g[b, c] / (2 eps), zero elsewhere;
// without bounds both land in grad_x.  One thread per row b (C is the number of classes).
__global__ __launch_bounds__(256) void margin_backward_kernel(const float* __restrict__ g,
                                                              const long long* __restrict__ targets, int B, int C,
                                                              float eps, float* __restrict__ grad_x,
                                                              float* __restrict__ grad_lower,
                                                              float* __restrict__ grad_upper) {
    const int b = blockIdx.x * 256 + threadIdx.x;
    if (b >= B) return;
    const long long tl = targets[b];
    const int t = tl < 0 || tl >= C ? -1 : (int)tl;  // a label outside the classes: no target column to write
    const float inv = 1.0f / (2.0f * eps);
    float sum = 0.f;
    for (int c = 0; c < C; c++) {
        const float v = c == t ? 0.f : g[(long)b * C + c] * inv;
        sum += v;
        if (grad_x != nullptr) grad_x[(long)b * C + c] = -v;
        if (grad_lower != nullptr) grad_lower[(long)b * C + c] = -v;
        if (grad_upper != nullptr) grad_upper[(long)b * C + c] = 0.f;
    }
    if (t < 0) return;
    if (grad_x != nullptr) grad_x[(long)b * C + t] = sum;
    if (grad_upper != nullptr) grad_upper[(long)b * C + t] = sum;
}

// One workgroup.  Every thread takes rows b = tid, tid + 1024, ...: row maximum (first index on ties) and row sum of
// relu(m); the rows' values are added over the workgroup in a fixed order (per-thread partials, butterfly, 16 wave
// sums in order).  argmax[b] = the class the maximum sits at, -1 when no margin is positive.
__global__ __launch_bounds__(1024) void hinge_forward_kernel(const float* __restrict__ margin, int B, int C, float mix,
                                                             float* __restrict__ loss, int* __restrict__ argmax) {
    __shared__ float part[2][16];
    float smax = 0.f, ssum = 0.f;
    for (int b = threadIdx.x; b < B; b += 1024) {
        float best = 0.f, rs = 0.f;
        int at = -1;
        for (int c = 0; c < C; c++) {
            // relu that lets NaN through, and a maximum that NaN wins, as torch's clamp(min=0) and max do in the
            // reference's loss: diverged activations or the NaN row of an out-of-range label must reach the loss
            const float m = margin[(long)b * C + c];
            const float r = m > 0.f ? m : (m != m ? m : 0.f);
            rs += r;
            if (r > best || (r != r && best == best)) { best = r; at = c; }
        }
        argmax[b] = at;
        smax += best;
        ssum += rs;
    }
#pragma unroll
    for (int d = 32; d >= 1; d >>= 1) {
        smax += __shfl_xor(smax, d, 64);
        ssum += __shfl_xor(ssum, d, 64);
    }
    if ((threadIdx.x & 63) == 0) { part[0][threadIdx.x >> 6] = smax; part[1][threadIdx.x >> 6] = ssum; }
    __syncthreads();
    if (threadIdx.x == 0) {
        float a = 0.f, s = 0.f;
        for (int q = 0; q < 16; q++) { a += part[0][q]; s += part[1][q]; }
        loss[0] = (1.0f - mix) * a / (float)B + mix * s / ((float)B * (float)C);
    }
}

// grad_margin[b, c] = g * [m > 0] * ((1 - mix) / B * [c == argmax[b]] + mix / (B * C))
__global__ __launch_bounds__(256) void hinge_backward_kernel(const float* __restrict__ margin, const int* __restrict__ argmax,
                                                             const float* __restrict__ grad_loss, int B, int C, float mix,
                                                             float* __restrict__ grad_margin) {
    const long i = (long)blockIdx.x * 256 + threadIdx.x;
    if (i >= (long)B * C) return;
    const int b = (int)(i / C), c = (int)(i - (long)b * C);
    const float g = grad_loss[0];
    const float w = (c == argmax[b] ? (1.0f - mix) / (float)B : 0.f) + mix / ((float)B * (float)C);
    grad_margin[i] = margin[i] > 0.f ? g * w : 0.f;
}

}  // namespace ndist

using namespace ndist;

extern "C" {

int ndist_margin_forward(const float* x, const float* lower, const float* upper, const long long* targets, int B, int C,
                         float eps, float* margin, ndist_stream_t stream) {
    if (targets == nullptr || margin == nullptr || (x == nullptr && (lower == nullptr || upper == nullptr))) return NDIST_ERR_NULL_POINTER;
    if (B <= 0 || C <= 0 || !(eps > 0.f)) return NDIST_ERR_BAD_SHAPE;
    const long n = (long)B * C;
    hipLaunchKernelGGL(margin_forward_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, (hipStream_t)stream, x, lower,
                       upper, targets, B, C, eps, margin);
    return hip_failed(hipGetLastError()) ? NDIST_ERR_HIP : NDIST_OK;
}

int ndist_margin_backward(const float* grad_margin, const long long* targets, int B, int C, float eps, float* grad_x,
                          float* grad_lower, float* grad_upper, ndist_stream_t stream) {
    if (grad_margin == nullptr || targets == nullptr) return NDIST_ERR_NULL_POINTER;
    if (B <= 0 || C <= 0 || !(eps > 0.f)) return NDIST_ERR_BAD_SHAPE;
    hipLaunchKernelGGL(margin_backward_kernel, dim3((unsigned)((B + 255) / 256)), dim3(256), 0, (hipStream_t)stream,
                       grad_margin, targets, B, C, eps, grad_x, grad_lower, grad_upper);
    return hip_failed(hipGetLastError()) ? NDIST_ERR_HIP : NDIST_OK;
}

int ndist_hinge_forward(const float* margin, int B, int C, float mix, float* loss, int* argmax, ndist_stream_t stream) {
    if (margin == nullptr || loss == nullptr || argmax == nullptr) return NDIST_ERR_NULL_POINTER;
    if (B <= 0 || C <= 0) return NDIST_ERR_BAD_SHAPE;
    hipLaunchKernelGGL(hinge_forward_kernel, dim3(1), dim3(1024), 0, (hipStream_t)stream, margin, B, C, mix, loss, argmax);
    return hip_failed(hipGetLastError()) ? NDIST_ERR_HIP : NDIST_OK;
}

int ndist_hinge_backward(const float* margin, const int* argmax, const float* grad_loss, int B, int C, float mix,
                         float* grad_margin, ndist_stream_t stream) {
    if (margin == nullptr || argmax == nullptr || grad_loss == nullptr || grad_margin == nullptr) return NDIST_ERR_NULL_POINTER;
    if (B <= 0 || C <= 0) return NDIST_ERR_BAD_SHAPE;
    const long n = (long)B * C;
    hipLaunchKernelGGL(hinge_backward_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, (hipStream_t)stream, margin,
                       argmax, grad_loss, B, C, mix, grad_margin);
    return hip_failed(hipGetLastError()) ? NDIST_ERR_HIP : NDIST_OK;
}

}  // extern "C"
