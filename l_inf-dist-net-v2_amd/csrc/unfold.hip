// Patch extraction for the convolutional distance layer: [B, C, H, W] -> [B, C*kh*kw, OH*OW], the layout the
// distance kernels take, and its adjoint.  The reference calls torch.nn.functional.unfold for this
// (core/modules/norm_dist.py:93-102), which on this platform launches one small kernel per sample; here the whole
// batch is one launch, the output (the large side) is written with 16-byte stores, and the adjoint gathers, so it
// needs neither atomics nor a zero fill.  Both are pure memory traffic.
#include "ndist_common.h"

namespace ndist {

// one thread: 4 consecutive output positions (same output row when OW % 4 == 0, checked by the launcher for VEC)
template <bool VEC>
__global__ __launch_bounds__(256) void unfold_kernel(const float* __restrict__ x, float* __restrict__ out,
                                                     const UnfoldGeom u, long nquad) {
    const long q = (long)blockIdx.x * 256 + threadIdx.x;
    if (q >= nquad) return;
    const int L = u.OH * u.OW;
    const int lq = VEC ? L / 4 : (L + 3) / 4;
    const int l0 = (int)(q % lq) * 4;
    long r = q / lq;
    const int j = (int)(r % u.kw);
    r /= u.kw;
    const int i = (int)(r % u.kh);
    r /= u.kh;  // r = b * C + c
    const float* __restrict__ img = x + r * u.H * u.W;
    float v[4];
#pragma unroll
    for (int t = 0; t < 4; t++) {
        const int l = l0 + t;
        const int oh = l / u.OW, ow = l - oh * u.OW;
        const int h = oh * u.sh - u.ph + i * u.dh, w = ow * u.sw - u.pw + j * u.dw;
        v[t] = (l < L && h >= 0 && h < u.H && w >= 0 && w < u.W) ? img[(long)h * u.W + w] : 0.f;
    }
    float* dst = out + ((r * u.kh + i) * u.kw + j) * L + l0;
    if (VEC) {
        *reinterpret_cast<float4*>(dst) = make_float4(v[0], v[1], v[2], v[3]);
    } else {
#pragma unroll
        for (int t = 0; t < 4; t++)
            if (l0 + t < L) dst[t] = v[t];
    }
}

// adjoint: every input element sums the patch entries it was copied to
__global__ __launch_bounds__(256) void fold_kernel(const float* __restrict__ gout, float* __restrict__ gx,
                                                   const UnfoldGeom u, long total) {
    const long e = (long)blockIdx.x * 256 + threadIdx.x;
    if (e >= total) return;
    const int w = (int)(e % u.W);
    long r = e / u.W;
    const int h = (int)(r % u.H);
    r /= u.H;  // r = b * C + c
    const int L = u.OH * u.OW;
    const float* __restrict__ col = gout + r * u.kh * u.kw * L;
    float acc = 0.f;
    for (int i = 0; i < u.kh; i++) {
        const int hn = h + u.ph - i * u.dh;
        if (hn < 0 || hn % u.sh != 0) continue;
        const int oh = hn / u.sh;
        if (oh >= u.OH) continue;
        for (int j = 0; j < u.kw; j++) {
            const int wn = w + u.pw - j * u.dw;
            if (wn < 0 || wn % u.sw != 0) continue;
            const int ow = wn / u.sw;
            if (ow >= u.OW) continue;
            acc += col[(long)(i * u.kw + j) * L + oh * u.OW + ow];
        }
    }
    gx[e] = acc;
}

// The patches as rows: out[m][k] with m = (b, oh, ow) and k = (c, i, j), k contiguous -- the transpose of the unfolded
// tensor, which is what the fused finite-p backward reads (lanes over k).  A workgroup owns one output row oh of one
// sample and CC channels: it stages the kh image rows those patches read (whole rows, coalesced) in LDS as
// strip[i][c][w], then writes, for every ow, the CC * kh * kw values of the row as one contiguous run.  Index
// arithmetic by float-reciprocal divisions (all operands below 2^22, checked by the launcher).
__global__ __launch_bounds__(256) void patch_rows_kernel(const float* __restrict__ x, float* __restrict__ out,
                                                         const UnfoldGeom u, int CC, int ncb, int vec4, float inv_w,
                                                         float inv_ccw, float inv_taps, float inv_kw) {
    extern __shared__ float strip[];  // [kh][CC][WP], WP = W | 1: neighbouring channels in different banks; then the
                                      // offsets of the block's CC * taps values inside the strip
    const int WP = u.W | 1;
    int* __restrict__ tapoff = reinterpret_cast<int*>(strip + u.kh * CC * WP);
    unsigned id = blockIdx.x;
    const int cb = (int)(id % (unsigned)ncb);
    id /= (unsigned)ncb;
    const int oh = (int)(id % (unsigned)u.OH), b = (int)(id / (unsigned)u.OH);
    const int c0 = cb * CC, ncl = min(CC, u.C - c0);
    const int taps = u.kh * u.kw, L = u.OH * u.OW;
    const long K = (long)u.C * taps;
    const int ccw = CC * u.W;
    for (int idx = threadIdx.x; idx < u.kh * ccw; idx += 256) {
        const int i = small_div(idx, ccw, inv_ccw), rem = idx - i * ccw;
        const int cl = small_div(rem, u.W, inv_w), wc = rem - cl * u.W;
        const int h = oh * u.sh - u.ph + i * u.dh;
        strip[(i * CC + cl) * WP + wc] =
            (cl < ncl && (unsigned)h < (unsigned)u.H) ? x[(((long)b * u.C + c0 + cl) * u.H + h) * u.W + wc] : 0.f;
    }
    // value kk of a run: strip offset of its row start and its column shift, worked out once per workgroup
    for (int kk = threadIdx.x; kk < CC * taps; kk += 256) {
        const int cl = small_div(kk, taps, inv_taps), tap = kk - cl * taps;
        const int i = small_div(tap, u.kw, inv_kw), j = tap - i * u.kw;
        tapoff[kk] = ((i * CC + cl) * WP << 8) | (j * u.dw);  // (the launcher keeps the shift below 256)
    }
    __syncthreads();
    const int run = ncl * taps;  // contiguous floats per output position
    float* __restrict__ dst = out + ((long)b * L + (long)oh * u.OW) * K + (long)c0 * taps;
    auto value = [&](int ow, int kk) {
        const int t = tapoff[kk];
        const int wc = ow * u.sw - u.pw + (t & 0xff);
        return (unsigned)wc < (unsigned)u.W ? strip[(t >> 8) + wc] : 0.f;
    };
    if (vec4) {  // run and K are multiples of four and out is 16-byte aligned: one store per four values
        const int run4 = run >> 2;
        const float inv_run4 = 1.0f / (float)run4;
        for (int idx = threadIdx.x; idx < u.OW * run4; idx += 256) {
            const int ow = small_div(idx, run4, inv_run4), kk = (idx - ow * run4) * 4;
            *reinterpret_cast<float4*>(dst + (long)ow * K + kk) =
                make_float4(value(ow, kk), value(ow, kk + 1), value(ow, kk + 2), value(ow, kk + 3));
        }
    } else {
        const float inv_run = 1.0f / (float)run;
        for (int idx = threadIdx.x; idx < u.OW * run; idx += 256) {
            const int ow = small_div(idx, run, inv_run), kk = idx - ow * run;
            dst[(long)ow * K + kk] = value(ow, kk);
        }
    }
}

// Adjoint of the above: gx[b, c, h, w] = sum over the taps (i, j) that read this pixel of g[m(b, oh, ow)][(c, i, j)].
// A workgroup owns 64 channels x 32 pixels of one image row; its threads run over the channels first, so that the
// reads of one tap (36 bytes apart for a 3 x 3 window) and of the neighbouring pixels' taps fall into the same cache
// lines, and the sums turn around in LDS for writes that run along w.  UNIT: both strides are 1 (no divisions).
// The taps are added in a fixed order: reproducible.
template <bool UNIT>
__global__ __launch_bounds__(256) void fold_rows_kernel(const float* __restrict__ g, float* __restrict__ gx,
                                                        const UnfoldGeom u) {
    __shared__ float tile[64][33];
    const int nwb = (u.W + 31) / 32, ncb = (u.C + 63) / 64;
    unsigned id = blockIdx.x;
    const int wb = (int)(id % (unsigned)nwb);
    id /= (unsigned)nwb;
    const int cb = (int)(id % (unsigned)ncb);
    id /= (unsigned)ncb;
    const int h = (int)(id % (unsigned)u.H), b = (int)(id / (unsigned)u.H);
    const int taps = u.kh * u.kw, L = u.OH * u.OW;
    const long K = (long)u.C * taps;
    const int cl = threadIdx.x & 63, c = cb * 64 + cl;
    const float* __restrict__ gb = g + (long)b * L * K + (long)(c < u.C ? c : 0) * taps;
    for (int wl = threadIdx.x >> 6; wl < 32; wl += 4) {
        const int w = wb * 32 + wl;
        float acc = 0.f;
        if (c < u.C && w < u.W) {
            for (int i = 0; i < u.kh; i++) {
                const int hn = h + u.ph - i * u.dh;
                int oh = hn;
                if (!UNIT) {
                    if (hn < 0 || hn % u.sh != 0) continue;
                    oh = hn / u.sh;
                }
                if ((unsigned)oh >= (unsigned)u.OH) continue;
                for (int j = 0; j < u.kw; j++) {
                    const int wn = w + u.pw - j * u.dw;
                    int ow = wn;
                    if (!UNIT) {
                        if (wn < 0 || wn % u.sw != 0) continue;
                        ow = wn / u.sw;
                    }
                    if ((unsigned)ow >= (unsigned)u.OW) continue;
                    acc += gb[(long)(oh * u.OW + ow) * K + i * u.kw + j];
                }
            }
        }
        tile[cl][wl] = acc;
    }
    __syncthreads();
    for (int idx = threadIdx.x; idx < 64 * 32; idx += 256) {
        const int cc = idx >> 5, wl = idx & 31;
        const int c2 = cb * 64 + cc, w = wb * 32 + wl;
        if (c2 < u.C && w < u.W) gx[(((long)b * u.C + c2) * u.H + h) * u.W + w] = tile[cc][wl];
    }
}

// The same sums from fewer, wider loads.  The kw taps of one window row lie side by side in memory, so a thread first
// adds, for one position and one channel, the taps of those window rows that reach image row h (4 * kw bytes per
// load, and which window rows reach h is the same for the whole workgroup), and leaves its kw sums in LDS; a pixel is
// then the sum of one tap from each of kw neighbouring positions.  KW: the window's width, 0 = any (one tap per
// load).  Fixed order of additions: reproducible.
template <int KW, bool UNIT>
__global__ __launch_bounds__(256) void fold_rows_taps_kernel(const float* __restrict__ g, float* __restrict__ gx,
                                                             const UnfoldGeom u, const int now, const int pitch) {
    extern __shared__ float part[];  // [64 channels][pitch >= now * kw]
    const int nwb = (u.W + 31) / 32, ncb = (u.C + 63) / 64;
    unsigned id = blockIdx.x;
    const int wb = (int)(id % (unsigned)nwb);
    id /= (unsigned)nwb;
    const int cb = (int)(id % (unsigned)ncb);
    id /= (unsigned)ncb;
    const int h = (int)(id % (unsigned)u.H), b = (int)(id / (unsigned)u.H);
    const int kw = KW ? KW : u.kw, taps = u.kh * kw, L = u.OH * u.OW;
    const long K = (long)u.C * taps;
    // first position whose window reaches the block's first pixel column
    const int lo = wb * 32 + u.pw - (kw - 1) * u.dw;
    const int ow0 = lo <= 0 ? 0 : (UNIT ? lo : (lo + u.sw - 1) / u.sw);
    const int cl = threadIdx.x & 63, c = cb * 64 + cl;
    if (c < u.C) {
        const float* __restrict__ gb = g + (long)b * L * K + (long)c * taps;
        for (int ol = threadIdx.x >> 6; ol < now; ol += 4) {
            const int ow = ow0 + ol;
            if (ow >= u.OW) break;
            float p[KW ? KW : 1];
#pragma unroll
            for (int j = 0; j < (KW ? KW : 1); j++) p[j] = 0.f;
            if (KW) {
                for (int i = 0; i < u.kh; i++) {
                    const int hn = h + u.ph - i * u.dh;
                    int oh = hn;
                    if (!UNIT) {
                        if (hn < 0 || hn % u.sh != 0) continue;
                        oh = hn / u.sh;
                    }
                    if ((unsigned)oh >= (unsigned)u.OH) continue;
                    const float* __restrict__ src = gb + (long)(oh * u.OW + ow) * K + i * KW;
#pragma unroll
                    for (int j = 0; j < KW; j++) p[j] += src[j];
                }
#pragma unroll
                for (int j = 0; j < KW; j++) part[cl * pitch + ol * KW + j] = p[j];
            } else {
                for (int j = 0; j < kw; j++) {
                    float acc = 0.f;
                    for (int i = 0; i < u.kh; i++) {
                        const int hn = h + u.ph - i * u.dh;
                        int oh = hn;
                        if (!UNIT) {
                            if (hn < 0 || hn % u.sh != 0) continue;
                            oh = hn / u.sh;
                        }
                        if ((unsigned)oh >= (unsigned)u.OH) continue;
                        acc += gb[(long)(oh * u.OW + ow) * K + i * kw + j];
                    }
                    part[cl * pitch + ol * kw + j] = acc;
                }
            }
        }
    }
    __syncthreads();
    for (int idx = threadIdx.x; idx < 64 * 32; idx += 256) {
        const int cc = idx >> 5, w = wb * 32 + (idx & 31);
        const int c2 = cb * 64 + cc;
        if (c2 >= u.C || w >= u.W) continue;
        float acc = 0.f;
#pragma unroll
        for (int j = 0; j < (KW ? KW : kw); j++) {
            const int wn = w + u.pw - j * u.dw;
            int ow = wn;
            if (!UNIT) {
                if (wn < 0 || wn % u.sw != 0) continue;
                ow = wn / u.sw;
            }
            if ((unsigned)ow >= (unsigned)u.OW) continue;
            acc += part[cc * pitch + (ow - ow0) * kw + j];
        }
        gx[(((long)b * u.C + c2) * u.H + h) * u.W + w] = acc;
    }
}

int launch_fold_rows(const float* g, const UnfoldGeom& u, float* gx, hipStream_t st) {
    const long blocks = (long)u.B * u.H * ((u.C + 63) / 64) * ((u.W + 31) / 32);
    if (blocks >= (1L << 31)) return 2;
    // positions whose windows reach a block of 32 pixel columns
    const long now = (31 + (long)(u.kw - 1) * u.dw) / u.sw + 2, pitch = (now * u.kw) | 1;
    if (u.kw >= 2 && 64 * pitch * sizeof(float) <= 64 * 1024) {
        const size_t lds = 64 * (size_t)pitch * sizeof(float);
        const bool unit = u.sh == 1 && u.sw == 1;
#define NDIST_FOLD_TAPS(KW, UNIT) \
    hipLaunchKernelGGL((fold_rows_taps_kernel<KW, UNIT>), dim3((unsigned)blocks), dim3(256), lds, st, g, gx, u, (int)now, \
                       (int)pitch)
        if (u.kw == 3 && unit) NDIST_FOLD_TAPS(3, true);
        else if (u.kw == 3) NDIST_FOLD_TAPS(3, false);
        else if (unit) NDIST_FOLD_TAPS(0, true);
        else NDIST_FOLD_TAPS(0, false);
#undef NDIST_FOLD_TAPS
        return hip_failed(hipGetLastError()) ? 4 : 0;
    }
    if (u.sh == 1 && u.sw == 1) hipLaunchKernelGGL(fold_rows_kernel<true>, dim3((unsigned)blocks), dim3(256), 0, st, g, gx, u);
    else hipLaunchKernelGGL(fold_rows_kernel<false>, dim3((unsigned)blocks), dim3(256), 0, st, g, gx, u);
    return hip_failed(hipGetLastError()) ? 4 : 0;
}

bool patch_rows_applies(const UnfoldGeom& u) {
    const int taps = u.kh * u.kw;
    int CC = 8192 / (u.kh * (u.W | 1));
    CC = CC > u.C ? u.C : CC;
    if (CC >= 4 && CC < u.C) CC &= ~3;
    if (CC < 1 || (long)u.kh * CC * u.W >= (1L << 22) || (long)u.OW * CC * taps >= (1L << 22)) return false;
    if ((long)(u.kw - 1) * u.dw >= 256 || (long)CC * taps > 8192) return false;  // packed tap offsets, 32 KB of them at most
    return (long)u.B * u.OH * ((u.C + CC - 1) / CC) < (1L << 31);
}

// returns -1 (nothing launched) when the geometry does not fit the kernel: the caller unfolds and transposes then
int launch_patch_rows(const float* x, const UnfoldGeom& u, float* out, hipStream_t st) {
    const int taps = u.kh * u.kw;
    int CC = 8192 / (u.kh * (u.W | 1));  // 32 KB of LDS for the strip
    CC = CC > u.C ? u.C : CC;
    if (CC >= 4 && CC < u.C) CC &= ~3;  // whole quads of channels: every run of a workgroup then allows 16-byte stores
    if (CC < 1 || (long)u.kh * CC * u.W >= (1L << 22) || (long)u.OW * CC * taps >= (1L << 22)) return -1;
    if ((long)(u.kw - 1) * u.dw >= 256 || (long)CC * taps > 8192) return -1;
    const int ncb = (u.C + CC - 1) / CC;
    const long blocks = (long)u.B * u.OH * ncb;
    if (blocks >= (1L << 31)) return -1;
    // 16-byte stores need every run of a workgroup to start and end on a multiple of four floats
    const int vec4 = (CC * taps) % 4 == 0 && (u.C * taps) % 4 == 0 && (uintptr_t)out % 16 == 0;
    hipLaunchKernelGGL(patch_rows_kernel, dim3((unsigned)blocks), dim3(256),
                       ((size_t)u.kh * CC * (u.W | 1) + (size_t)CC * taps) * sizeof(float), st, x,
                       out, u, CC, ncb, vec4, 1.0f / (float)u.W, 1.0f / (float)(CC * u.W), 1.0f / (float)taps,
                       1.0f / (float)u.kw);
    return hip_failed(hipGetLastError()) ? 4 : 0;
}

int launch_unfold(const float* x, const UnfoldGeom& u, float* out, hipStream_t st) {
    const int L = u.OH * u.OW;
    const bool vec = L % 4 == 0 && (uintptr_t)out % 16 == 0;
    const long nquad = (long)u.B * u.C * u.kh * u.kw * (vec ? L / 4 : (L + 3) / 4);
    const long blocks = (nquad + 255) / 256;
    if (blocks >= (1L << 31)) return 2;
    KernelTimer timer(st);
    if (vec) hipLaunchKernelGGL(unfold_kernel<true>, dim3((unsigned)blocks), dim3(256), 0, st, x, out, u, nquad);
    else hipLaunchKernelGGL(unfold_kernel<false>, dim3((unsigned)blocks), dim3(256), 0, st, x, out, u, nquad);
    return hip_failed(hipGetLastError()) ? 4 : 0;
}

int launch_fold(const float* gout, const UnfoldGeom& u, float* gx, hipStream_t st) {
    const long total = (long)u.B * u.C * u.H * u.W;
    const long blocks = (total + 255) / 256;
    if (blocks >= (1L << 31)) return 2;
    KernelTimer timer(st);
    hipLaunchKernelGGL(fold_kernel, dim3((unsigned)blocks), dim3(256), 0, st, gout, gx, u, total);
    return hip_failed(hipGetLastError()) ? 4 : 0;
}

}  // namespace ndist
