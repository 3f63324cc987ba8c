// Mean shift and bias of a distance layer in one launch (fully connected layout, shift_fused_kernel) or two to
// three: what follows every operator call in the reference's layers (core/modules/norm_dist.py:35-38 -> core/modules/basic_modules.py:121-132): the per-channel
// batch mean of x (training; the running mean in evaluation) is subtracted from x and from both interval bounds, the
// moving average is updated, and the layer's bias is added.  With torch primitives this is a reduction, an in-place
// update and an elementwise kernel per tensor; here:
//   1. colsum_partial_kernel   partial[rb][j] = sum over the rows b of block rb of t1[b][j] (+ t2 + t3),  j = (c, hw)
//   2. mean_finalize_kernel    per channel: the partials in a fixed order -> mean, moving average, column sum
//   3. shift_apply_kernel      y = t - mean[c] + bias1[c] + bias2[c] for up to three tensors
// Evaluation needs only the third.  The backward of the training path is the same three steps on the gradients:
// grad_x = g_x - mean_c(g_x + g_lower + g_upper), and the column sums are the bias gradients.  Sums are taken in a
// fixed order (no atomics): results repeat bit for bit.
#include "../../include/norm_dist_hip.h"
#include "ndist_common.h"

namespace ndist {

constexpr int kShiftRowsPerBlock = 32;

__global__ __launch_bounds__(256) void colsum_partial_kernel(const float* __restrict__ t1, const float* __restrict__ t2,
                                                             const float* __restrict__ t3, int B, long N,
                                                             float* __restrict__ partial) {
    const long j = (long)blockIdx.x * 256 + threadIdx.x;
    if (j >= N) return;
    const int b0 = blockIdx.y * kShiftRowsPerBlock, b1 = min(B, b0 + kShiftRowsPerBlock);
    float s = 0.f;
    for (int b = b0; b < b1; b++) {
        float v = t1[(long)b * N + j];
        if (t2 != nullptr) v += t2[(long)b * N + j];
        if (t3 != nullptr) v += t3[(long)b * N + j];
        s += v;
    }
    partial[(long)blockIdx.y * N + j] = s;
}

// one wave per channel: lane l takes the items l, l + 64, ... of the channel's nrb * HW partial sums, then the lanes
// are combined by a butterfly; every step has a fixed order
__global__ __launch_bounds__(64) void mean_finalize_kernel(const float* __restrict__ partial, int nrb, int C, int HW,
                                                           float inv_count, float momentum,
                                                           float* __restrict__ running_mean, float* __restrict__ mean_out,
                                                           float* __restrict__ colsum_out) {
    const int c = blockIdx.x, lane = threadIdx.x;
    const long N = (long)C * HW;
    float s = 0.f;
    for (int i = lane; i < nrb * HW; i += 64) {
        const int rb = i / HW, hw = i - rb * HW;
        s += partial[(long)rb * N + (long)c * HW + hw];
    }
#pragma unroll
    for (int d = 32; d >= 1; d >>= 1) s += __shfl_xor(s, d, 64);
    if (lane == 0) {
        const float mean = s * inv_count;
        if (mean_out != nullptr) mean_out[c] = mean;
        if (colsum_out != nullptr) colsum_out[c] = s;
        if (running_mean != nullptr) running_mean[c] = running_mean[c] * (1.0f - momentum) + mean * momentum;
    }
}

// y_i = t_i - mean[c] + bias1[c] + bias2[c]; VEC: 0 scalar, 1 four consecutive elements of one channel (HW % 4 == 0),
// 2 four consecutive channels (HW == 1, C % 4 == 0)
template <int VEC>
__global__ __launch_bounds__(256) void shift_apply_kernel(const float* __restrict__ t1, const float* __restrict__ t2,
                                                          const float* __restrict__ t3, float* __restrict__ y1,
                                                          float* __restrict__ y2, float* __restrict__ y3,
                                                          const float* __restrict__ mean, const float* __restrict__ bias1,
                                                          const float* __restrict__ bias2, long total, int C, int HW) {
    const long i = ((long)blockIdx.x * 256 + threadIdx.x) * (VEC ? 4 : 1);
    if (i >= total) return;
    auto shift_of = [&](int c) -> float {
        float sft = mean != nullptr ? mean[c] : 0.f;
        if (bias1 != nullptr) sft -= bias1[c];
        if (bias2 != nullptr) sft -= bias2[c];
        return sft;
    };
    const int c = (int)((i / HW) % C);
    if (VEC == 0) {
        const float sft = shift_of(c);
        if (t1 != nullptr) y1[i] = t1[i] - sft;
        if (t2 != nullptr) y2[i] = t2[i] - sft;
        if (t3 != nullptr) y3[i] = t3[i] - sft;
    } else {
        float4 sft;
        if (VEC == 1) {
            const float v = shift_of(c);
            sft = make_float4(v, v, v, v);
        } else {
            sft = make_float4(shift_of(c), shift_of(c + 1), shift_of(c + 2), shift_of(c + 3));
        }
        auto one = [&](const float* __restrict__ t, float* __restrict__ y) {
            if (t == nullptr) return;
            const float4 v = *reinterpret_cast<const float4*>(t + i);
            *reinterpret_cast<float4*>(y + i) = make_float4(v.x - sft.x, v.y - sft.y, v.z - sft.z, v.w - sft.w);
        };
        one(t1, y1);
        one(t2, y2);
        one(t3, y3);
    }
}

static bool aligned16(const void* p) { return p == nullptr || (uintptr_t)p % 16 == 0; }

// All three steps in one launch for the fully connected layout (HW == 1, C % 4 == 0): a workgroup owns 32 channels
// (one 128-byte line per batch row), adds its rows up in a fixed order (thread (r, q) the rows r, r + 32, ... of
// four channels, then the 32 partial sums in order), writes mean / column sum / moving average and goes over its
// rows a second time to subtract (that pass finds them in the L2).  t2 and t3 only join the sum (the adjoint: the
// gradients of the two bounds).
constexpr int kFusedCols = 32;
__global__ __launch_bounds__(256) void shift_fused_kernel(const float* __restrict__ t1, const float* __restrict__ t2,
                                                          const float* __restrict__ t3, float* __restrict__ y1, int B, int C,
                                                          float inv_count, float momentum, float* __restrict__ running_mean,
                                                          float* __restrict__ mean_out, float* __restrict__ colsum_out,
                                                          const float* __restrict__ bias1, const float* __restrict__ bias2) {
    __shared__ float4 part[32][8];
    const int q = threadIdx.x & 7, r = threadIdx.x >> 3;
    const int c = blockIdx.x * kFusedCols + q * 4;
    const bool live = c < C;
    float4 s = make_float4(0.f, 0.f, 0.f, 0.f);
    if (live) {
#pragma unroll 4
        for (int b = r; b < B; b += 32) {
            float4 v = *reinterpret_cast<const float4*>(t1 + (long)b * C + c);
            if (t2 != nullptr) {
                const float4 u = *reinterpret_cast<const float4*>(t2 + (long)b * C + c);
                v = make_float4(v.x + u.x, v.y + u.y, v.z + u.z, v.w + u.w);
            }
            if (t3 != nullptr) {
                const float4 u = *reinterpret_cast<const float4*>(t3 + (long)b * C + c);
                v = make_float4(v.x + u.x, v.y + u.y, v.z + u.z, v.w + u.w);
            }
            s = make_float4(s.x + v.x, s.y + v.y, s.z + v.z, s.w + v.w);
        }
    }
    part[r][q] = s;
    __syncthreads();
    float4 tot = make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
    for (int i = 0; i < 32; i++) {
        const float4 v = part[i][q];
        tot = make_float4(tot.x + v.x, tot.y + v.y, tot.z + v.z, tot.w + v.w);
    }
    if (!live) return;
    const float4 mean = make_float4(tot.x * inv_count, tot.y * inv_count, tot.z * inv_count, tot.w * inv_count);
    if (r == 0) {
        if (mean_out != nullptr) *reinterpret_cast<float4*>(mean_out + c) = mean;
        if (colsum_out != nullptr) *reinterpret_cast<float4*>(colsum_out + c) = tot;
        if (running_mean != nullptr) {
            const float k = 1.0f - momentum;
            running_mean[c] = running_mean[c] * k + mean.x * momentum;
            running_mean[c + 1] = running_mean[c + 1] * k + mean.y * momentum;
            running_mean[c + 2] = running_mean[c + 2] * k + mean.z * momentum;
            running_mean[c + 3] = running_mean[c + 3] * k + mean.w * momentum;
        }
    }
    if (y1 == nullptr) return;
    float4 sft = mean;
    if (bias1 != nullptr) sft = make_float4(sft.x - bias1[c], sft.y - bias1[c + 1], sft.z - bias1[c + 2], sft.w - bias1[c + 3]);
    if (bias2 != nullptr) sft = make_float4(sft.x - bias2[c], sft.y - bias2[c + 1], sft.z - bias2[c + 2], sft.w - bias2[c + 3]);
#pragma unroll 4
    for (int b = r; b < B; b += 32) {
        const float4 v = *reinterpret_cast<const float4*>(t1 + (long)b * C + c);
        *reinterpret_cast<float4*>(y1 + (long)b * C + c) = make_float4(v.x - sft.x, v.y - sft.y, v.z - sft.z, v.w - sft.w);
    }
}

static bool fused_applies(const float* t1, const float* t2, const float* t3, const float* y1, const float* m1, const float* m2,
                          int C, int HW) {
    return HW == 1 && C % 4 == 0 && aligned16(t1) && aligned16(t2) && aligned16(t3) && aligned16(y1) && aligned16(m1) &&
           aligned16(m2);
}
static int launch_fused(const float* t1, const float* t2, const float* t3, float* y1, int B, int C, float momentum,
                        float* running_mean, float* mean_out, float* colsum_out, const float* b1, const float* b2,
                        hipStream_t st) {
    hipLaunchKernelGGL(shift_fused_kernel, dim3(ceil_div(C, kFusedCols)), dim3(256), 0, st, t1, t2, t3, y1, B, C,
                       1.0f / (float)B, momentum, running_mean, mean_out, colsum_out, b1, b2);
    return hip_failed(hipGetLastError()) ? 4 : 0;
}

static int launch_apply(const float* t1, const float* t2, const float* t3, float* y1, float* y2, float* y3,
                        const float* mean, const float* b1, const float* b2, int B, int C, int HW, hipStream_t st) {
    const long total = (long)B * C * HW;
    const bool al = aligned16(t1) && aligned16(t2) && aligned16(t3) && aligned16(y1) && aligned16(y2) && aligned16(y3);
    const int vec = !al ? 0 : (HW % 4 == 0 ? 1 : (HW == 1 && C % 4 == 0 ? 2 : 0));
    const long items = vec ? total / 4 : total;
    const dim3 grid((unsigned)((items + 255) / 256));
    if (vec == 1) hipLaunchKernelGGL(shift_apply_kernel<1>, grid, dim3(256), 0, st, t1, t2, t3, y1, y2, y3, mean, b1, b2, total, C, HW);
    else if (vec == 2) hipLaunchKernelGGL(shift_apply_kernel<2>, grid, dim3(256), 0, st, t1, t2, t3, y1, y2, y3, mean, b1, b2, total, C, HW);
    else hipLaunchKernelGGL(shift_apply_kernel<0>, grid, dim3(256), 0, st, t1, t2, t3, y1, y2, y3, mean, b1, b2, total, C, HW);
    return hip_failed(hipGetLastError()) ? 4 : 0;
}

// column means of t1 (+ t2 + t3) into mean_out (and the sums into colsum_out), moving average updated when given
static int launch_colmean(const float* t1, const float* t2, const float* t3, int B, int C, int HW, float momentum,
                          float* running_mean, float* mean_out, float* colsum_out, hipStream_t st) {
    const long N = (long)C * HW;
    const int nrb = ceil_div(B, kShiftRowsPerBlock);
    float* partial = nullptr;
    NDIST_HIP_TRY(scratch_alloc((void**)&partial, (size_t)nrb * N * sizeof(float), st));
    hipLaunchKernelGGL(colsum_partial_kernel, dim3((unsigned)((N + 255) / 256), nrb), dim3(256), 0, st, t1, t2, t3, B, N,
                       partial);
    int rc = hip_failed(hipGetLastError()) ? 4 : 0;
    if (!rc) {
        hipLaunchKernelGGL(mean_finalize_kernel, dim3(C), dim3(64), 0, st, partial, nrb, C, HW,
                           1.0f / ((float)B * (float)HW), momentum, running_mean, mean_out, colsum_out);
        rc = hip_failed(hipGetLastError()) ? 4 : 0;
    }
    if (hip_failed(scratch_free(partial, st)) && !rc) rc = 4;
    return rc;
}

}  // namespace ndist

using namespace ndist;

extern "C" {

int ndist_mean_shift_forward(const float* x, const float* lower, const float* upper, int B, int C, int HW, int training,
                             float momentum, float* running_mean, const float* bias1, const float* bias2,
                             float* mean_out, float* y, float* y_lower, float* y_upper, ndist_stream_t stream) {
    if ((x == nullptr) != (y == nullptr) || (lower == nullptr) != (y_lower == nullptr) ||
        (upper == nullptr) != (y_upper == nullptr))
        return NDIST_ERR_NULL_POINTER;
    if (x == nullptr && lower == nullptr && upper == nullptr) return NDIST_ERR_NULL_POINTER;
    if (B <= 0 || C <= 0 || HW <= 0 || (long long)B * C * HW > 0x7fffffffLL) return NDIST_ERR_BAD_SHAPE;
    hipStream_t st = (hipStream_t)stream;
    const float* mean = running_mean;
    if (training) {
        // the batch mean of x (the reference requires x in training, core/modules/basic_modules.py:123)
        if (x == nullptr || mean_out == nullptr) return NDIST_ERR_NULL_POINTER;
        if (lower == nullptr && upper == nullptr && fused_applies(x, nullptr, nullptr, y, mean_out, nullptr, C, HW))
            return launch_fused(x, nullptr, nullptr, y, B, C, momentum, running_mean, mean_out, nullptr, bias1, bias2, st);
        if (int rc = launch_colmean(x, nullptr, nullptr, B, C, HW, momentum, running_mean, mean_out, nullptr, st)) return rc;
        mean = mean_out;
    }  // evaluation without a running mean: biases only
    return launch_apply(x, lower, upper, y, y_lower, y_upper, mean, bias1, bias2, B, C, HW, st);
}

int ndist_mean_shift_backward(const float* grad_y, const float* grad_y_lower, const float* grad_y_upper, int B, int C,
                              int HW, int training, float* grad_x, float* colsum_out, float* mean_scratch,
                              ndist_stream_t stream) {
    if (B <= 0 || C <= 0 || HW <= 0 || (long long)B * C * HW > 0x7fffffffLL) return NDIST_ERR_BAD_SHAPE;
    // the first non-null gradient leads the sum
    const float* g[3] = {grad_y, grad_y_lower, grad_y_upper};
    const float* lead = nullptr;
    const float* rest[2] = {nullptr, nullptr};
    int nrest = 0;
    for (int i = 0; i < 3; i++) {
        if (g[i] == nullptr) continue;
        if (lead == nullptr) lead = g[i];
        else rest[nrest++] = g[i];
    }
    if (lead == nullptr) return NDIST_ERR_NULL_POINTER;
    hipStream_t st = (hipStream_t)stream;
    if (!training && colsum_out == nullptr) return NDIST_OK;  // evaluation: grad_x is grad_y itself, nothing to do
    if (mean_scratch == nullptr) return NDIST_ERR_NULL_POINTER;
    if (training && grad_x != nullptr && lead == grad_y &&
        fused_applies(lead, rest[0], rest[1], grad_x, mean_scratch, colsum_out, C, HW))
        return launch_fused(lead, rest[0], rest[1], grad_x, B, C, 0.f, nullptr, mean_scratch, colsum_out, nullptr, nullptr, st);
    if (int rc = launch_colmean(lead, rest[0], rest[1], B, C, HW, 0.f, nullptr, mean_scratch, colsum_out, st)) return rc;
    if (!training || grad_x == nullptr) return NDIST_OK;
    if (grad_y == nullptr) {
        // x's own output received no gradient: grad_x = -mean alone; expressed as 0 - mean through the bias slot
        return NDIST_ERR_NULL_POINTER;
    }
    return launch_apply(grad_y, nullptr, nullptr, grad_x, nullptr, nullptr, mean_scratch, nullptr, nullptr, B, C, HW, st);
}

}  // extern "C"
