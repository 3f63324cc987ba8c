// Forward of the finite-p distance  out = (sum_k |x - w|^p)^(1/p).
// Replaces norm_dist<ip>::forward and ::forward_with_max of the reference
// (core/cuda/norm_dist_cuda.cu:35-236,511-564; algorithm choice core/cuda/norm_dist.cpp:40-64):
//   integral p in 1..10   plain sum, |t|^p by repeated multiplication (the reference does so up to 8 and uses
//                         pow for 9 and 10; both are the same function of t to well below the 1e-5 tolerance)
//   other p <= 10         plain sum, |t|^p = exp2(p * log2 |t|) on the hardware transcendentals
//   p > 10                sum of (|t| / m)^p with a running maximum m per output, rescaled whenever m grows, so that
//                         large p neither overflows nor underflows; starts from m = 1e-10 with the phantom term 1
//   caller-supplied m     forward_with_max: the same sum with m read from a tensor
// The plain sum is floored at FLT_MIN before the root, as the reference does.
#include <atomic>

#include "fwd_norm_ops.h"
#include "seed_outputs.h"

namespace ndist {

// Device-side probe of the |x - w| distribution, used by the backward to choose between its plain and its
// term-skipping kernel (whose lanes run over k, so that what matters there is the plain fraction of pairs that
// count): on a sample of outputs, the number of pairs above the drop threshold thr * max_k |x - w|.  One workgroup
// per sampled output; counts are added to gate[0].
constexpr int kProbeOutputs = 128;
__global__ __launch_bounds__(256) void norm_probe_kernel(const float* __restrict__ x, const float* __restrict__ w,
                                                         const Geom s, float thr, int* __restrict__ gate) {
    __shared__ float red[4];
    __shared__ int cnt[4];
    const int i = blockIdx.x, lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int m = (int)(((long)i * 7919 + 13) % s.M), n = (int)(((long)i * 104729 + 7) % s.COg), g = i % s.G;
    const int b = m / s.HW, hw = m - b * s.HW;
    const float* __restrict__ xp = x + x_off(s, b, g, 0, hw);
    const float* __restrict__ wp = w + w_off(s, g, n, 0);
    float mx = 0.f;
    for (int k = threadIdx.x; k < s.CIg; k += 256) mx = fmaxf(mx, fabsf(xp[(long)k * s.HW] - wp[k]));
#pragma unroll
    for (int d = 32; d >= 1; d >>= 1) mx = fmaxf(mx, __shfl_xor(mx, d, 64));
    if (lane == 0) red[wave] = mx;
    __syncthreads();
    mx = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
    const float t = mx * thr;
    int c = 0;
    for (int k = threadIdx.x; k < s.CIg; k += 256) c += fabsf(xp[(long)k * s.HW] - wp[k]) > t ? 1 : 0;
#pragma unroll
    for (int d = 32; d >= 1; d >>= 1) c += __shfl_xor(c, d, 64);
    if (lane == 0) cnt[wave] = c;
    __syncthreads();
    if (threadIdx.x == 0) atomicAdd(gate, cnt[0] + cnt[1] + cnt[2] + cnt[3]);
}

// Probe of the forward skipping operator.  What that operator costs depends on how often some pair of a wave's step
// (8 rows x 8 * TN columns x 2 k) counts, not on how many pairs count: when the w rows are nearly equal, or a few
// large weights decide the maxima, the pairs that count line up over the columns or the rows and the steps that do
// the expensive work are few; when they are independent almost every step holds one.  So the probe counts steps, on
// a sample of blocks of 8 consecutive rows x 40 consecutive columns.  Two small kernels, the k range split over
// workgroups so that neither takes more than a few microseconds: the first leaves the 320 maxima of every block in
// scratch memory, the second counts the pairs of k in which any of the 640 pairs exceeds thr * (its maximum).
constexpr int kProbeBlocks = 16;
constexpr int kProbeRowsB = 8, kProbeColsB = 40, kProbeOutB = kProbeRowsB * kProbeColsB;
constexpr int kProbeChunk = 128;  // k per workgroup
constexpr int kProbePitch = kProbeChunk + 1;

// Stages the block's rows of x and w for one k chunk in LDS (zero beyond CIg) and returns the block's coordinates.
__device__ __forceinline__ void probe_stage(const float* __restrict__ x, const float* __restrict__ w, const Geom& s,
                                            float* __restrict__ xs, float* __restrict__ ws, int blk, int k0) {
    const int g = blk % s.G;
    const int nmb = s.M / kProbeRowsB > 0 ? s.M / kProbeRowsB : 1, nnb = s.COg / kProbeColsB > 0 ? s.COg / kProbeColsB : 1;
    const int m0 = (int)(((long)blk * 7919 + 13) % nmb) * kProbeRowsB;
    const int n0 = (int)(((long)blk * 104729 + 7) % nnb) * kProbeColsB;
    for (int i = threadIdx.x; i < (kProbeRowsB + kProbeColsB) * kProbeChunk; i += 256) {
        const int r = i / kProbeChunk, kk = i - r * kProbeChunk, k = k0 + kk;
        float v = 0.f;
        if (r < kProbeRowsB) {
            const int m = min(m0 + r, s.M - 1), b = m / s.HW, hw = m - b * s.HW;
            if (k < s.CIg) v = x[x_off(s, b, g, k, hw)];
            xs[r * kProbePitch + kk] = v;
        } else {
            const int n = min(n0 + r - kProbeRowsB, s.COg - 1);
            if (k < s.CIg) v = w[w_off(s, g, n, k)];
            ws[(r - kProbeRowsB) * kProbePitch + kk] = v;
        }
    }
}

// grid (blocks, k chunks): maxima[blk][o] = max_k |x - w| of output o = row * 40 + column of the block
// (atomic maximum on the bit patterns of non-negative floats; the buffer starts at zero)
__global__ __launch_bounds__(256) void norm_probe_max_kernel(const float* __restrict__ x, const float* __restrict__ w,
                                                             const Geom s, float* __restrict__ maxima) {
    __shared__ float xs[kProbeRowsB * kProbePitch], ws[kProbeColsB * kProbePitch];
    const int blk = blockIdx.x, k0 = blockIdx.y * kProbeChunk;
    probe_stage(x, w, s, xs, ws, blk, k0);
    __syncthreads();
    for (int o = threadIdx.x; o < kProbeOutB; o += 256) {
        const float* xr = xs + (o / kProbeColsB) * kProbePitch;
        const float* wr = ws + (o % kProbeColsB) * kProbePitch;
        float mx = 0.f;
        for (int kk = 0; kk < kProbeChunk; kk++) mx = fmaxf(mx, fabsf(xr[kk] - wr[kk]));
        atomicMax(reinterpret_cast<unsigned*>(maxima) + blk * kProbeOutB + o, __float_as_uint(mx));
    }
}

// grid (blocks, k chunks): gate[0] += number of pairs of k of the chunk in which some output of the block has a pair
// above thr * (its maximum).  Every thread keeps one bit per pair of k for its outputs; the bits are OR-ed over the
// block.
__global__ __launch_bounds__(256) void norm_probe_count_kernel(const float* __restrict__ x, const float* __restrict__ w,
                                                               const Geom s, const float* __restrict__ maxima, float thr,
                                                               int* __restrict__ gate) {
    __shared__ float xs[kProbeRowsB * kProbePitch], ws[kProbeColsB * kProbePitch];
    __shared__ unsigned long long part[4];
    static_assert(kProbeChunk / 2 <= 64, "one bit per pair of k");
    const int blk = blockIdx.x, k0 = blockIdx.y * kProbeChunk;
    probe_stage(x, w, s, xs, ws, blk, k0);
    __syncthreads();
    unsigned long long bits = 0;
    for (int o = threadIdx.x; o < kProbeOutB; o += 256) {
        const float* xr = xs + (o / kProbeColsB) * kProbePitch;
        const float* wr = ws + (o % kProbeColsB) * kProbePitch;
        const float t = maxima[blk * kProbeOutB + o] * thr;
        for (int q = 0; q < kProbeChunk / 2; q++) {
            const float e = fmaxf(fabsf(xr[2 * q] - wr[2 * q]), fabsf(xr[2 * q + 1] - wr[2 * q + 1]));
            bits |= e > t ? 1ull << q : 0ull;
        }
    }
#pragma unroll
    for (int d = 32; d >= 1; d >>= 1) bits |= __shfl_xor(bits, d, 64);
    if ((threadIdx.x & 63) == 0) part[threadIdx.x >> 6] = bits;
    __syncthreads();
    if (threadIdx.x == 0) {
        bits = part[0] | part[1] | part[2] | part[3];
        const int npair = min(kProbeChunk, s.CIg - k0) / 2;  // pairs of the chunk that exist
        if (npair < 64) bits &= (1ull << npair) - 1;
        const int c = __popcll(bits);
        if (c != 0) atomicAdd(gate, c);
    }
}

int fill_zero(float* p, long n, hipStream_t st);  // bwd_norm_c.hip

// Pre-pass of the skipping operators over the rows of a matrix with k contiguous (x with HW == 1, or w), one wave per
// row: the element of largest magnitude (signed; NaN when the row holds a NaN) and its k, and the largest magnitude
// inside every 32-wide k-tile (tile_max[row][ntile]).
struct SeedSide {
    const float* x;
    const float* x2;  // interval bounds: second array of the same shape, the larger magnitude of the two counts
    long rows;
    int K;
    float* seed;
    int32_t* seed_k;
    float* tile_max;
    // interval bounds, optional: per row the largest max(-lower, upper) and the largest max(lower, -upper) over k,
    // inverted boxes collapsed to their midpoint first (NaN when the row holds a NaN)
    float* out_hi;
    float* out_lo;
};
template <int CTRL>
__device__ __forceinline__ float lane_swap(float v) {  // data-parallel-primitive move: no LDS traffic
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xf, 0xf, true));
}
// The row's elements through 16-byte loads (1 KiB per wave and instruction), ten loads in flight per lane: a wave
// alone keeps 10 KiB on its way.  The loads are unconditional (addresses behind the row's end fall back on its last
// four k): a load under a per-lane condition is split into four 4-byte ones.  The tile maxima of a pass go through
// LDS so that they leave in whole lines.  BOX: two arrays (interval bounds), the larger magnitude of the two counts.
template <bool BOX>
__device__ __forceinline__ void seed_row_wide(const float* __restrict__ xp, const float* __restrict__ xq, int K, int ntile,
                                              float* __restrict__ tm, int lane, float& best, float& val, int& bk,
                                              bool& bad, float& far_hi, float& far_lo) {
    constexpr int U = BOX ? 5 : 10;
    __shared__ float stage_all[4][8 * U];
    float* stage = stage_all[threadIdx.x >> 6];
    for (int k0 = 0; k0 < K; k0 += 256 * U) {
        float4 a4[U], b4[BOX ? U : 1];
#pragma unroll
        for (int u = 0; u < U; u++) {
            const int k = min(k0 + 256 * u + 4 * lane, K - 4);
            a4[u] = *reinterpret_cast<const float4*>(xp + k);
            if constexpr (BOX) b4[u] = *reinterpret_cast<const float4*>(xq + k);
        }
#pragma unroll
        for (int u = 0; u < U; u++) {
            const int k = k0 + 256 * u + 4 * lane;
            if (k0 + 256 * u >= K) break;  // wave-uniform
            float local = 0.f;  // largest magnitude of my four k: they lie in one tile, 8 lanes share a tile
            if (k < K) {
                float v[4] = {a4[u].x, a4[u].y, a4[u].z, a4[u].w};
                const float sum4 = (v[0] + v[1]) + (v[2] + v[3]);
                bad |= sum4 != sum4;
                if constexpr (BOX) {
                    const float v2[4] = {b4[u].x, b4[u].y, b4[u].z, b4[u].w};
                    const float sum4b = (v2[0] + v2[1]) + (v2[2] + v2[3]);
                    bad |= sum4b != sum4b;
#pragma unroll
                    for (int j = 0; j < 4; j++) {
                        float lo = v[j], up = v2[j];
                        if (lo > up) lo = up = (lo + up) * 0.5f;
                        far_hi = fmaxf(far_hi, fmaxf(-lo, up));
                        far_lo = fmaxf(far_lo, fmaxf(lo, -up));
                        v[j] = fabsf(v2[j]) > fabsf(v[j]) ? v2[j] : v[j];
                    }
                }
#pragma unroll
                for (int j = 0; j < 4; j++) {
                    local = fmaxf(local, fabsf(v[j]));
                    if (fabsf(v[j]) > best) { best = fabsf(v[j]); val = v[j]; bk = k + j; }
                }
            }
            local = fmaxf(local, lane_swap<0xB1>(local));   // quad_perm [1, 0, 3, 2]
            local = fmaxf(local, lane_swap<0x4E>(local));   // quad_perm [2, 3, 0, 1]
            local = fmaxf(local, lane_swap<0x141>(local));  // row_half_mirror
            if ((lane & 7) == 0) stage[8 * u + (lane >> 3)] = local;
        }
        __builtin_amdgcn_wave_barrier();
        const int t0 = k0 >> 5, nt = min(8 * U, ntile - t0);
        for (int t = lane; t < nt; t += 64) tm[t0 + t] = stage[t];
        __builtin_amdgcn_wave_barrier();
    }
}

__device__ __forceinline__ void norm_seed_row(const SeedSide& sd, long r, int ntile) {
    const int lane = threadIdx.x & 63;
    const int K = sd.K;
    const float* __restrict__ x = sd.x;
    const float* __restrict__ xp = x + r * K;
    const float* __restrict__ xq = sd.x2 != nullptr ? sd.x2 + r * K : nullptr;  // second array: magnitudes of both count
    float* __restrict__ tm = sd.tile_max + r * ntile;
    float best = -1.f, val = 0.f;
    int bk = 0;
    bool bad = false;  // a NaN in the row (or +inf next to -inf): the pair at the row's seed may not exist
    float far_hi = -__builtin_inff(), far_lo = -__builtin_inff();
    if (K % 4 == 0 && (uintptr_t)x % 16 == 0 && (uintptr_t)sd.x2 % 16 == 0) {
        if (xq == nullptr) seed_row_wide<false>(xp, xq, K, ntile, tm, lane, best, val, bk, bad, far_hi, far_lo);
        else seed_row_wide<true>(xp, xq, K, ntile, tm, lane, best, val, bk, bad, far_hi, far_lo);
    } else {
        for (int k0 = 0; k0 < K; k0 += 64) {
            const int k = k0 + lane;
            float local = 0.f;  // 32 lanes share a tile
            if (k < K) {
                float v = xp[k];
                bad |= v != v;
                if (xq != nullptr) {
                    const float v2 = xq[k];
                    bad |= v2 != v2;
                    float lo = v, up = v2;
                    if (lo > up) lo = up = (lo + up) * 0.5f;
                    far_hi = fmaxf(far_hi, fmaxf(-lo, up));
                    far_lo = fmaxf(far_lo, fmaxf(lo, -up));
                    v = fabsf(v2) > fabsf(v) ? v2 : v;
                }
                local = fabsf(v);
                if (fabsf(v) > best) { best = fabsf(v); val = v; bk = k; }
            }
#pragma unroll
            for (int d = 1; d < 32; d <<= 1) local = fmaxf(local, __shfl_xor(local, d, 64));
            if ((lane & 31) == 0 && k < K) tm[k >> 5] = local;
        }
    }
#pragma unroll
    for (int d = 32; d >= 1; d >>= 1) {
        const float ob = __shfl_xor(best, d, 64), ov = __shfl_xor(val, d, 64);
        const int ok = __shfl_xor(bk, d, 64);
        if (ob > best) { best = ob; val = ov; bk = ok; }
    }
    // a row with a NaN is marked by a NaN seed value: consumers that form pairs with it drop them like any NaN pair
    if (__builtin_amdgcn_ballot_w64(bad) != 0) val = __builtin_nanf("");
    if (lane == 0) { sd.seed[r] = val; sd.seed_k[r] = bk; }
    if (sd.out_hi != nullptr) {
#pragma unroll
        for (int d = 32; d >= 1; d >>= 1) {
            far_hi = fmaxf(far_hi, __shfl_xor(far_hi, d, 64));
            far_lo = fmaxf(far_lo, __shfl_xor(far_lo, d, 64));
        }
        if (lane == 0) {
            sd.out_hi[r] = val == val ? far_hi : val;
            sd.out_lo[r] = val == val ? far_lo : val;
        }
    }
}


// Blocks [0, nblocks_a) serve side a, the next nblocks_b side b, the others side c (four rows per block).  Does
// nothing when the probe's count (gate[0]) says that the skipping operator will not run.  `zero`, `zero2`: four ints
// each, cleared for the kernels that follow.
__global__ __launch_bounds__(256) void norm_seed_kernel(const SeedSide a, const SeedSide b, const SeedSide c,
                                                        int nblocks_a, int nblocks_b, int ntile,
                                                        const int* __restrict__ gate, int gate_limit,
                                                        int* __restrict__ zero, int* __restrict__ zero2) {
    if (zero != nullptr && blockIdx.x == 0 && threadIdx.x < 4) zero[threadIdx.x] = 0;
    if (zero2 != nullptr && blockIdx.x == 0 && threadIdx.x >= 64 && threadIdx.x < 68) zero2[threadIdx.x - 64] = 0;
    if (gate != nullptr && gate[0] >= gate_limit) return;
    const int blk = (int)blockIdx.x;
    const int side = blk < nblocks_a ? 0 : (blk < nblocks_a + nblocks_b ? 1 : 2);
    const SeedSide& sd = side == 0 ? a : (side == 1 ? b : c);
    const long r = (long)(blk - (side == 0 ? 0 : (side == 1 ? nblocks_a : nblocks_a + nblocks_b))) * 4 + (threadIdx.x >> 6);
    if (r >= sd.rows) return;  // whole waves leave: the shuffles stay wave-uniform
    norm_seed_row(sd, r, ntile);
}

// Seed of every output (seed_outputs.h), one workgroup per 64 rows x 64 columns of one group.
__global__ __launch_bounds__(256) void norm_seed_outputs_kernel(const float* __restrict__ x, const float* __restrict__ w,
                                                                const Geom s, const OutputSeedJob job,
                                                                const int* __restrict__ gate, int gate_limit) {
    __shared__ float tile[kSeedTileFloats];
    if (gate != nullptr && gate[0] >= gate_limit) return;
    norm_seed_outputs_block(x, w, s, job, blockIdx.x, tile);
}

__global__ __launch_bounds__(256) void bound_seed_outputs_kernel(const float* __restrict__ xl, const float* __restrict__ xu,
                                                                 const float* __restrict__ w, const Geom s,
                                                                 const OutputSeedJob job, const int* __restrict__ gate,
                                                                 int gate_limit) {
    __shared__ float tiles[2 * kSeedTileFloats];
    if (gate != nullptr && gate[0] >= gate_limit) return;
    bound_seed_outputs_block(xl, xu, w, s, job, blockIdx.x, tiles);
}

size_t seed_scratch_floats(const Geom& s) {
    const size_t rows = (size_t)s.M * s.G, wrows = (size_t)s.COg * s.G, total = (size_t)s.M * s.COg * s.G;
    return (2 + (size_t)ceil_div(s.CIg, 32)) * (rows + wrows) + total;
}

size_t bound_seed_scratch_floats(const Geom& s) {
    return seed_scratch_floats(s) + (size_t)s.M * s.COg * s.G + 2 * (size_t)s.M * s.G;
}

size_t weight_seed_floats(const Geom& s) {
    return (2 + (size_t)ceil_div(s.CIg, 32)) * ((size_t)s.COg * s.G);
}

WeightSeeds weight_seeds_at(float* base, const Geom& s) {
    const long wrows = (long)s.COg * s.G;
    WeightSeeds ws{};
    ws.seed_w = base;
    ws.seed_wk = reinterpret_cast<int32_t*>(base + wrows);
    ws.tile_w = reinterpret_cast<float*>(ws.seed_wk + wrows);
    return ws;
}

int launch_weight_seeds(const float* w, const Geom& s, float* base, const int* gate, int gate_limit, hipStream_t st,
                        WeightSeeds* out) {
    const long wrows = (long)s.COg * s.G;
    const int ntile = ceil_div(s.CIg, 32);
    *out = weight_seeds_at(base, s);
    const SeedSide sw{w, nullptr, wrows, s.CIg, out->seed_w, out->seed_wk, out->tile_w, nullptr, nullptr};
    hipLaunchKernelGGL(norm_seed_kernel, dim3((unsigned)((wrows + 3) / 4)), dim3(256), 0, st, sw, SeedSide{}, SeedSide{},
                       (int)((wrows + 3) / 4), 0, ntile, gate, gate_limit, (int*)nullptr, (int*)nullptr);
    return hip_failed(hipGetLastError()) ? 4 : 0;
}

// Where the results of the row pre-pass lie in an operator's seed scratch (`base`), and the two sides of its launch:
// the rows of x (of the box when x2 is given) and, unless `wpre` brings them, the rows of w.
static void layout_row_seeds(const float* x, const float* w, const Geom& s, float* base, const float* x2,
                             const WeightSeeds* wpre, SeedBuffers* out, SeedSide* side_x, SeedSide* side_w) {
    const long rows = (long)s.M * s.G, wrows = (long)s.COg * s.G, total = (long)s.M * s.COg * s.G;
    const int ntile = ceil_div(s.CIg, 32);
    float* seed_x = base;
    int32_t* seed_k = reinterpret_cast<int32_t*>(seed_x + rows);
    float* seed_w = reinterpret_cast<float*>(seed_k + rows);
    int32_t* seed_wk = reinterpret_cast<int32_t*>(seed_w + wrows);
    float* seed = reinterpret_cast<float*>(seed_wk + wrows);
    float* tile_x = seed + total;
    float* tile_w = tile_x + rows * ntile;
    float* const after_tiles = tile_w + wrows * ntile;
    if (wpre != nullptr) {
        seed_w = wpre->seed_w;
        seed_wk = wpre->seed_wk;
        tile_w = wpre->tile_w;
    }
    // (interval bounds: the two extra row statistics lie behind the second seed array)
    float* far_hi = x2 != nullptr ? after_tiles + total : nullptr;
    float* far_lo = x2 != nullptr ? far_hi + rows : nullptr;
    *side_x = SeedSide{x, x2, rows, s.CIg, seed_x, seed_k, tile_x, far_hi, far_lo};
    *side_w = SeedSide{w, nullptr, wpre != nullptr ? 0 : wrows, s.CIg, seed_w, seed_wk, tile_w, nullptr, nullptr};
    out->seed = seed;
    out->seed2 = x2 != nullptr ? after_tiles : nullptr;  // interval bounds: the second seed array lies behind the tile bounds
    out->tile_x = tile_x;
    out->tile_w = tile_w;
    out->ntile = ntile;
    out->far_hi = far_hi;
    out->far_lo = far_lo;
    out->seed_x = seed_x;
    out->seed_k = seed_k;
    out->seed_w = seed_w;
    out->seed_wk = seed_wk;
}

int launch_row_seeds(const float* x, const float* w, const Geom& s, float* base, const int* gate, int gate_limit,
                     hipStream_t st, SeedBuffers* out, const float* x2, const WeightSeeds* wpre, int* zero) {
    SeedSide sx{}, sw{};
    layout_row_seeds(x, w, s, base, x2, wpre, out, &sx, &sw);
    // one launch for the rows of x and (unless done before) the rows of w
    const int nbx = (int)((sx.rows + 3) / 4), nbw = (int)((sw.rows + 3) / 4);
    hipLaunchKernelGGL(norm_seed_kernel, dim3((unsigned)(nbx + nbw)), dim3(256), 0, st, sx, sw, SeedSide{}, nbx, nbw,
                       out->ntile, gate, gate_limit, zero, (int*)nullptr);
    return hip_failed(hipGetLastError()) ? 4 : 0;
}

// The row pre-passes of a layer's distance (x) and of its interval bounds (the box xl, xu) in one launch, with the
// rows of w unless `wpre` brings them; both operators then read the same results for w.
int launch_joint_row_seeds(const float* x, const float* xl, const float* xu, const float* w, const Geom& s, float* base,
                           float* base_box, const WeightSeeds* wpre, hipStream_t st, SeedBuffers* out,
                           SeedBuffers* out_box, int* zero, int* zero_box) {
    SeedSide sx{}, sw{}, sb{}, unused{};
    layout_row_seeds(x, w, s, base, nullptr, wpre, out, &sx, &sw);
    const WeightSeeds shared{out->seed_w, out->seed_wk, out->tile_w};  // wherever the first layout put (or found) them
    layout_row_seeds(xl, w, s, base_box, xu, &shared, out_box, &sb, &unused);
    const int nbx = (int)((sx.rows + 3) / 4), nbb = (int)((sb.rows + 3) / 4), nbw = (int)((sw.rows + 3) / 4);
    hipLaunchKernelGGL(norm_seed_kernel, dim3((unsigned)(nbx + nbb + nbw)), dim3(256), 0, st, sx, sb, sw, nbx, nbb,
                       out->ntile, (const int*)nullptr, 0, zero, zero_box);
    return hip_failed(hipGetLastError()) ? 4 : 0;
}

int launch_output_seeds(const float* x, const float* w, const Geom& s, const SeedBuffers& sb, const int* gate,
                        int gate_limit, hipStream_t st, const float* x2) {
    const OutputSeedJob job = output_seed_job(s, sb);
    const dim3 grid((unsigned)((long)job.nmb * job.nnb * s.G));
    if (x2 == nullptr) hipLaunchKernelGGL(norm_seed_outputs_kernel, grid, dim3(256), 0, st, x, w, s, job, gate, gate_limit);
    else hipLaunchKernelGGL(bound_seed_outputs_kernel, grid, dim3(256), 0, st, x, x2, w, s, job, gate, gate_limit);
    return hip_failed(hipGetLastError()) ? 4 : 0;
}

int launch_seeds(const float* x, const float* w, const Geom& s, float* base, const int* gate, int gate_limit,
                 hipStream_t st, SeedBuffers* out, const float* x2, const WeightSeeds* wpre) {
    int rc = launch_row_seeds(x, w, s, base, gate, gate_limit, st, out, x2, wpre);
    const int ro = launch_output_seeds(x, w, s, *out, gate, gate_limit, st, x2);
    return rc ? rc : ro;
}

// Probe scratch: [0] the count (int), from float 4 on the maxima.  Zeroes it and leaves in [0] the number of sampled
// steps in which some pair counts; the sample has kProbeBlocks * (CIg / 2) steps, and the skipping operator is the
// faster one while fewer than about two thirds of them do.
constexpr size_t kProbeScratchFloats = 4 + (size_t)kProbeBlocks * kProbeOutB;
static int launch_norm_probe_steps(const float* x, const float* w, const Geom& s, float thr, float* scratch,
                                   hipStream_t st) {
    const int rc = fill_zero(scratch, (long)kProbeScratchFloats, st);
    if (rc) return rc;
    const dim3 grid(kProbeBlocks, ceil_div(s.CIg, kProbeChunk));
    hipLaunchKernelGGL(norm_probe_max_kernel, grid, dim3(256), 0, st, x, w, s, scratch + 4);
    if (hip_failed(hipGetLastError())) return 4;
    hipLaunchKernelGGL(norm_probe_count_kernel, grid, dim3(256), 0, st, x, w, s, scratch + 4, thr,
                       reinterpret_cast<int*>(scratch));
    return hip_failed(hipGetLastError()) ? 4 : 0;
}
static int norm_probe_steps_limit(const Geom& s) { return (int)(0.65 * kProbeBlocks * (s.CIg / 2)) + 1; }

// Zeroes gate[0] and adds to it the number of sampled pairs above thr * (their output's maximum); the sample has
// kProbeOutputs * CIg pairs.
int launch_norm_probe(const float* x, const float* w, const Geom& s, float thr, int* gate, hipStream_t st) {
    const int rc = fill_zero(reinterpret_cast<float*>(gate), 1, st);
    if (rc) return rc;
    hipLaunchKernelGGL(norm_probe_kernel, dim3(kProbeOutputs), dim3(256), 0, st, x, w, s, thr, gate);
    return hip_failed(hipGetLastError()) ? 4 : 0;
}
int norm_probe_limit(const Geom& s) { return (int)(0.025 * kProbeOutputs * s.CIg) + 1; }
static int env_mode(const char* name) {
    const char* v = getenv(name);
    return v == nullptr ? -1 : (v[0] == '0' ? 0 : 1);
}
// The overrides belong to the calling host thread (thread_local): a thread that never called the setter uses the
// value the environment gave at load time, and no thread can leave another one on a different kernel path.
static const int g_env_skip = env_mode("NORM_DIST_SKIP"), g_env_bounds = env_mode("NORM_DIST_BWD_BOUNDS");
static thread_local int t_skip_mode = g_env_skip, t_bounds_mode = g_env_bounds;
void set_skip_mode(int skip, int bounds) {
    t_skip_mode = skip < 0 ? g_env_skip : (skip ? 1 : 0);
    t_bounds_mode = bounds < 0 ? g_env_bounds : (bounds ? 1 : 0);
}
void get_skip_mode(int* skip, int* bounds) {
    *skip = t_skip_mode;
    *bounds = t_bounds_mode;
}
static int override_limit(int mode, int probed_limit) { return mode < 0 ? probed_limit : (mode == 0 ? 0 : 0x7fffffff); }
int skip_override_limit(int probed_limit) { return override_limit(t_skip_mode, probed_limit); }
int bounds_override_limit(int probed_limit) { return override_limit(t_bounds_mode, probed_limit); }
bool skip_forced_on() { return t_skip_mode == 1; }

// ---- one-pass normalised sum with a per-row scale (OpRowScaled) ------------------------------------------

// Largest magnitude of every row of x (rows_x rows of K values) and of w (rows_w rows): one wave per row.
__global__ __launch_bounds__(256) void row_absmax_kernel(const float* __restrict__ x, long rows_x,
                                                         const float* __restrict__ w, long rows_w, int K, int vec,
                                                         float* __restrict__ rx, float* __restrict__ rw) {
    const long r = (long)blockIdx.x * 4 + (threadIdx.x >> 6);
    const int lane = threadIdx.x & 63;
    if (r >= rows_x + rows_w) return;
    const float* __restrict__ row = r < rows_x ? x + r * K : w + (r - rows_x) * K;
    float m = 0.f;
    if (vec) {
        const float4* __restrict__ v = reinterpret_cast<const float4*>(row);
        for (int k = lane; k < K / 4; k += 64) {
            const float4 q = v[k];
            m = fmaxf(fmaxf(m, fmaxf(fabsf(q.x), fabsf(q.y))), fmaxf(fabsf(q.z), fabsf(q.w)));
        }
    } else {
        for (int k = lane; k < K; k += 64) m = fmaxf(m, fabsf(row[k]));
    }
#pragma unroll
    for (int d = 32; d >= 1; d >>= 1) m = fmaxf(m, __shfl_xor(m, d, 64));
    if (lane == 0) (r < rows_x ? rx[r] : rw[r - rows_x]) = m;
}

// c[r] = p * log2(max(rx[r] + max(rw), 1e-10)): every workgroup reduces rw for itself (a few thousand values).
__global__ __launch_bounds__(256) void row_scale_kernel(const float* __restrict__ rx, long rows_x,
                                                        const float* __restrict__ rw, long rows_w, float p,
                                                        float* __restrict__ c) {
    __shared__ float part[4];
    float m = 0.f;
    for (long n = threadIdx.x; n < rows_w; n += 256) m = fmaxf(m, rw[n]);
#pragma unroll
    for (int d = 32; d >= 1; d >>= 1) m = fmaxf(m, __shfl_xor(m, d, 64));
    if ((threadIdx.x & 63) == 0) part[threadIdx.x >> 6] = m;
    __syncthreads();
    m = fmaxf(fmaxf(part[0], part[1]), fmaxf(part[2], part[3]));
    const long r = (long)blockIdx.x * 256 + threadIdx.x;
    if (r < rows_x) c[r] = p * fast_log2(fmaxf(rx[r] + m, kEps));
}

// Outputs the one-pass kernel marked with -1 (sum below the safe range, or NaN): recomputed by one wave each with
// the exact maximum, as the two-pass operator does (maximum floored at 1e-10, its term added).  Fully connected
// layout only (HW == 1).
__global__ __launch_bounds__(256) void norm_fixup_kernel(const float* __restrict__ x, const float* __restrict__ w,
                                                         const Geom s, float p, float inv_p, float* __restrict__ out) {
    const int lane = threadIdx.x & 63;
    const long total = (long)s.M * s.COg * s.G;
    const int CO = s.COg * s.G, K = s.CIg;
    for (long base = ((long)blockIdx.x * 4 + (threadIdx.x >> 6)) * 64; base < total; base += (long)gridDim.x * 256) {
        const long o = base + lane;
        unsigned long long marked = __builtin_amdgcn_ballot_w64(o < total && out[o] < 0.f);
        while (marked != 0) {
            const int l = __builtin_ctzll(marked);
            marked &= marked - 1;
            const long oo = base + l;
            const int b = (int)(oo / CO), cn = (int)(oo - (long)b * CO), g = cn / s.COg;
            const float* __restrict__ xr = x + ((long)b * s.G + g) * K;
            const float* __restrict__ wr = w + (long)cn * K;
            float m = kEps;
            for (int k = lane; k < K; k += 64) m = fmaxf(m, fabsf(xr[k] - wr[k]));
#pragma unroll
            for (int d = 32; d >= 1; d >>= 1) m = fmaxf(m, __shfl_xor(m, d, 64));
            const float c = p * fast_log2(m);
            float sum = 0.f;
            for (int k = lane; k < K; k += 64) sum += fast_exp2(fmaf(p, fast_log2(fabsf(xr[k] - wr[k])), -c));
#pragma unroll
            for (int d = 32; d >= 1; d >>= 1) sum += __shfl_xor(sum, d, 64);
            sum += fast_exp2(p * fast_log2(kEps) - c);
            if (lane == 0) out[oo] = fast_exp2(fast_log2(sum) * inv_p) * m;
        }
    }
}

static const int g_env_scaled = env_mode("NORM_DIST_ROW_SCALE");
static thread_local int t_scaled_mode = g_env_scaled;
void set_scaled_mode(int mode) { t_scaled_mode = mode < 0 ? g_env_scaled : (mode ? 1 : 0); }
int scaled_mode() { return t_scaled_mode; }
// Up to p = 48 a scale 3.2 times the true maximum still keeps the sum above 2^-90; beyond, too many outputs would
// take the slow exact route on ordinary data.
constexpr float kMaxRowScaledP = 48.0f;
static bool row_scaled_applies(const Geom& s, float p) {
    const int mode = t_scaled_mode;
    if (mode == 0 || s.HW != 1 || !(p <= kMaxRowScaledP) || skinny_applies(s)) return false;
    return mode == 1 || (double)s.M * s.COg * s.G * s.CIg >= 2e7;
}
static size_t row_scaled_scratch_floats(const Geom& s) { return 2 * (size_t)s.M * s.G + (size_t)s.COg * s.G; }
// Queues the two scale kernels, the one-pass kernel and the pass over marked outputs; `scratch` holds
// row_scaled_scratch_floats(s) floats.  P carries the gate, if any, for the main kernel only.
static int launch_row_scaled(FwdParams P, float* scratch, hipStream_t st) {
    const Geom& s = P.s;
    const long rows_x = (long)s.M * s.G, rows_w = (long)s.COg * s.G;
    float* rx = scratch;
    float* c = rx + rows_x;
    float* rw = c + rows_x;
    const int vec = s.CIg % 4 == 0 && (reinterpret_cast<uintptr_t>(P.x) & 15) == 0 && (reinterpret_cast<uintptr_t>(P.w) & 15) == 0;
    hipLaunchKernelGGL(row_absmax_kernel, dim3((unsigned)((rows_x + rows_w + 3) / 4)), dim3(256), 0, st, P.x, rows_x, P.w,
                       rows_w, s.CIg, vec, rx, rw);
    hipLaunchKernelGGL(row_scale_kernel, dim3((unsigned)((rows_x + 255) / 256)), dim3(256), 0, st, rx, rows_x, rw, rows_w, P.p, c);
    if (hip_failed(hipGetLastError())) return 4;
    P.aux = c;
    const int rc = launch_fwd<OpRowScaled, CfgWide4, CfgBig, CfgSmall, CfgWide, CfgLow32, CfgLow16, CfgWide4H>(P, st);
    if (rc) return rc;
    const long total = rows_x * s.COg;
    const unsigned grid = (unsigned)std::min<long>((total + 255) / 256, 4096);
    hipLaunchKernelGGL(norm_fixup_kernel, dim3(grid), dim3(256), 0, st, P.x, P.w, s, P.p, P.inv_p, P.out);
    return hip_failed(hipGetLastError()) ? 4 : 0;
}

template <int IP>
static int launch_sum(const FwdParams& P, hipStream_t st) {
    if constexpr (IP == 8)  // (with the eight-waves-per-SIMD configurations as candidates 7 and 8, for measurements)
        return launch_fwd<OpSum<IP>, CfgWide4, CfgBig, CfgSmall, CfgWide, CfgLow32, CfgLow16, CfgWide4H, CfgOcc8, CfgOcc8W>(P, st);
    return launch_fwd<OpSum<IP>, CfgWide4, CfgBig, CfgSmall, CfgWide, CfgLow32, CfgLow16, CfgWide4H>(P, st);
}

int launch_norm_forward(const float* x, const float* w, const float* max_in, const Geom& s, float* out, float p,
                        hipStream_t st) {
    FwdParams P{};
    P.x = x;
    P.w = w;
    P.aux = max_in;
    P.out = out;
    P.s = s;
    P.p = p;
    P.inv_p = 1.0f / p;
    if (max_in != nullptr) return launch_fwd<OpNormalized<true>, CfgWideT, CfgMid, CfgSmall>(P, st);
    if (p > kMinNormalizedP) {
        // Large p: the skipping operator is up to three times faster when few of a wave's steps hold a pair near the
        // maximum, and up to 1.6 times slower than the plain one when most do.  For problems worth the three extra
        // launches a device-side probe counts such steps on a sample; both variants are queued and the probe's count
        // (below or above 65 % of the sampled steps) opens the gate of one of them.
        constexpr float kMinSkipP = 16.0f;  // below, the threshold 2^(-32/p) leaves almost nothing to skip
        const double pairs = (double)s.M * s.COg * s.G * s.CIg;
        const bool scaled = row_scaled_applies(s, p);  // the one-pass kernel stands in for the plain two-pass one
        if (p < kMinSkipP || (pairs < 2e8 && !skip_forced_on()) || skinny_applies(s)) {
            float* rs = nullptr;
            if (!scaled || scratch_alloc((void**)&rs, row_scaled_scratch_floats(s) * sizeof(float), st) != hipSuccess) {
                (void)hipGetLastError();
                return launch_fwd<OpNormalized<false>, CfgWideT, CfgMid, CfgSmall, CfgLow32, CfgLow16>(P, st);
            }
            int rc = launch_row_scaled(P, rs, st);
            if (hip_failed(scratch_free(rs, st)) && !rc) rc = 4;
            return rc;
        }
        P.thr = exp2f(-32.0f / p);
        P.inv_thr = 1.0f / P.thr;
        float* scratch = nullptr;  // probe scratch, then the seeds of the skipping operator (values, indices)
        const size_t nskip = kProbeScratchFloats + seed_scratch_floats(s);
        if (scratch_alloc((void**)&scratch, (nskip + (scaled ? row_scaled_scratch_floats(s) : 0)) * sizeof(float), st) != hipSuccess) {
            (void)hipGetLastError();  // no scratch (out of memory, or a stream under capture): the plain kernel needs none
            return launch_fwd<OpNormalized<false>, CfgWideT, CfgMid, CfgSmall, CfgLow32, CfgLow16>(P, st);
        }
        int* gate = reinterpret_cast<int*>(scratch);
        int rc = launch_norm_probe_steps(x, w, s, P.thr, scratch, st);
        P.gate = gate;
        P.gate_limit = skip_override_limit(norm_probe_steps_limit(s));
        // seeds only where k is the contiguous axis: in the conv layout the pre-passes cost what they save
        if (!rc && s.HW == 1) {
            SeedBuffers sb{};
            rc = launch_seeds(x, w, s, scratch + kProbeScratchFloats, gate, P.gate_limit, st, &sb);
            P.aux = sb.seed;
            P.tile_x = sb.tile_x;
            P.tile_w = sb.tile_w;
            P.ntile32 = sb.ntile;
        }
        KernelTimer timer(st);  // the variant that runs
        if (!rc) {
            P.gate_sense = 1;  // few pairs count: skip
            rc = launch_fwd<OpNormSkip<false>, CfgWideT, CfgMid, CfgSmall>(P, st);
        }
        if (!rc) {
            P.gate_sense = 0;
            P.aux = nullptr;
            rc = scaled ? launch_row_scaled(P, scratch + nskip, st) : launch_fwd<OpNormalized<false>, CfgWideT, CfgMid, CfgSmall, CfgLow32, CfgLow16>(P, st);
        }
        if (hip_failed(scratch_free(scratch, st)) && !rc) rc = 4;
        return rc;
    }
    if (p == (float)(int)p) {
        switch ((int)p) {
            case 1: return launch_sum<1>(P, st);
            case 2: return launch_sum<2>(P, st);
            case 3: return launch_sum<3>(P, st);
            case 4: return launch_sum<4>(P, st);
            case 5: return launch_sum<5>(P, st);
            case 6: return launch_sum<6>(P, st);
            case 7: return launch_sum<7>(P, st);
            case 8: return launch_sum<8>(P, st);
            case 9: return launch_sum<9>(P, st);
            case 10: return launch_sum<10>(P, st);
            default: break;
        }
    }
    return launch_sum<0>(P, st);
}

}  // namespace ndist
