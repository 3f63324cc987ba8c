// Second pass of the arg-max forward kernels of a convolutional layer called on images: turns the winning k-tile of
// every output into the arg-max code (reference semantics: core/cuda/inf_dist_cuda.cu:14-198 and
// core/cuda/bound_inf_dist_cuda.cu:15-238 keep the first k that attains the extremum, plus a sign flag).
//
// The sorted second pass (rescan_sorted.h) gathers a k-tile of patches through the patch geometry once per tile and
// workgroup, 36 times at 3 x 3 windows over 128 channels, with two barriers each.  Here a workgroup owns a few whole
// output rows of one sample and stages the image rows under their windows ONCE: all channels of the group, padding
// included as zeros, in LDS (70 KB for two output rows of a 32 x 32 image with 128 channels).  Every patch element
// of every position of the block is then one LDS read away — its address is a per-k table entry plus a per-position
// offset — so each output looks at its own winning tile directly: no sort, no barrier after the staging, no atomics.
// Four lanes (a quad) share an output: four consecutive k each, twice for tiles of 32 k.  A wave reads tile and target
// of 64 consecutive positions of one output channel with coalesced loads, hands them to its quads by quad
// permutations (no trip through the LDS crossbar), and writes the 64 codes back coalesced.
//
// BOUND: both interval outputs in one launch, and in one walk where they peak in the same tile, on the same staged
// pair of images, inverted boxes collapsed to their midpoint while staging (reference: core/cuda/bound_inf_dist_cuda.cu:63).
#pragma once
#include "ndist_common.h"
#include <algorithm>
#include <cstdlib>
#include <type_traits>

namespace ndist {

constexpr int kRiMaxSlots = 8;               // staged elements of one channel per lane: 64 * 8 floats per channel
constexpr int kRiLdsBudget = 150 * 1024;     // of the 160 KB of a compute unit
constexpr int kRiMaxK = 8192;

struct ImageRowBlocks {
    int R;         // output rows per workgroup
    int nrb;       // row blocks per sample
    int rows_in;   // image rows staged per channel: (R - 1) sh + (kh - 1) dh + 1
    int pitch;     // staged row length: W + 2 pw
    int E;         // rows_in * pitch, floats per channel
    int nt;        // number of k-tiles
    float inv_pitch, inv_ow;
};

template <bool BOUND, int KT>
__global__ __launch_bounds__(1024) void rescan_image_kernel(const float* __restrict__ x, const float* __restrict__ x2,
                                                            const float* __restrict__ w, const float* __restrict__ out1,
                                                            int32_t* __restrict__ pos1, const float* __restrict__ out2,
                                                            int32_t* __restrict__ pos2, const Geom s, const PatchMap pm,
                                                            const ImageRowBlocks rg, int w_vec) {
    extern __shared__ float lds[];
    constexpr uint32_t kNoKey = 0xffffffffu;
    static_assert(KT == 16 || KT == 32, "four lanes of four k cover a tile in one or two steps");
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6), nwave = (int)blockDim.x >> 6;
    unsigned id = blockIdx.x;
    const int rb = (int)(id % (unsigned)rg.nrb);
    id /= (unsigned)rg.nrb;
    const int g = (int)(id % (unsigned)s.G), b = (int)(id / (unsigned)s.G);
    const int cg = pm.cg, E = rg.E, K = s.CIg, OW = pm.OW, OH = s.HW / pm.OW;
    const int K4 = (K + 3) & ~3;
    int* __restrict__ tab = reinterpret_cast<int*>(lds);  // [K4]: tap of k as an offset in xs (16-byte aligned)
    float* __restrict__ xs = lds + K4;                     // [NX][cg][E]
    const int oh0 = rb * rg.R, nrow = min(rg.R, OH - oh0), npos = nrow * OW, hw0 = oh0 * OW;
    const int ih_base = oh0 * pm.sh - pm.ph;

    for (int k = tid; k < K4; k += (int)blockDim.x) {
        const int kc = min(k, K - 1);  // the entries that round K up to whole quads are never used for a hit
        const int cl = small_div(kc, pm.taps, pm.inv_taps), tap = kc - cl * pm.taps;
        const int ti = small_div(tap, pm.kw, pm.inv_kw), tj = tap - ti * pm.kw;
        tab[k] = cl * E + ti * pm.dh * rg.pitch + tj * pm.dw;
    }
    // ---- staging: a wave takes whole channels; what a lane fetches of a channel is the same for every channel
    {
        int goff[kRiMaxSlots];
        bool ok[kRiMaxSlots];
#pragma unroll
        for (int q = 0; q < kRiMaxSlots; q++) {
            const int e = lane + 64 * q;
            const int r = small_div(e, rg.pitch, rg.inv_pitch), col = e - r * rg.pitch;
            const int ih = ih_base + r, iw = col - pm.pw;
            ok[q] = e < E && (unsigned)ih < (unsigned)pm.H && (unsigned)iw < (unsigned)pm.W;
            goff[q] = ok[q] ? ih * pm.W + iw : 0;
        }
        const long plane = (long)pm.H * pm.W;
        const float* __restrict__ img1 = x + ((long)b * pm.C + (long)g * cg) * plane;
        const float* __restrict__ img2 = BOUND ? x2 + ((long)b * pm.C + (long)g * cg) * plane : nullptr;
#pragma unroll 2
        for (int c = wave; c < cg; c += nwave) {
            float v1[kRiMaxSlots], v2[kRiMaxSlots];
#pragma unroll
            for (int q = 0; q < kRiMaxSlots; q++) {
                if (64 * q < E) {  // uniform
                    v1[q] = img1[c * plane + goff[q]];
                    if (BOUND) v2[q] = img2[c * plane + goff[q]];
                }
            }
#pragma unroll
            for (int q = 0; q < kRiMaxSlots; q++) {
                const int e = lane + 64 * q;
                if (64 * q < E && e < E) {
                    float lo = ok[q] ? v1[q] : 0.f;
                    if (BOUND) {
                        float hi = ok[q] ? v2[q] : 0.f;
                        if (lo > hi) lo = hi = (lo + hi) * 0.5f;
                        xs[(cg + c) * E + e] = hi;
                    }
                    xs[c * E + e] = lo;
                }
            }
        }
    }
    __syncthreads();

    // ---- every output looks at its winning tile
    const int nmacro = (npos + 63) >> 6;  // blocks of 64 consecutive positions
    const int total = s.COg * nmacro;
    // BOUND: the lower and the upper output of a box usually peak in the same tile (always, when the box has the same
    // width everywhere): one walk over that tile then serves both; an upper output with a tile of its own gets a
    // second walk.
#pragma unroll 1
    for (int it = wave; it < total; it += nwave) {
        const int n = it / nmacro, p = (it - n * nmacro) * 64 + lane;
        const bool live = p < npos;
        int t1st = -1, t2nd = -1, poff = 0;
        float val1 = 0.f, val2 = 0.f;
        long o = 0;
        if (live) {
            o = y_off(s, b, g, n, hw0 + p);
            t1st = pos1[o];
            val1 = BOUND ? -out1[o] : out1[o];
            if (t1st < 0 || t1st >= rg.nt) t1st = -1;
            if constexpr (BOUND) {
                t2nd = pos2[o];
                val2 = out2[o];
                if (t2nd < 0 || t2nd >= rg.nt) t2nd = -1;
            }
            const int pr = small_div(p, OW, rg.inv_ow), pc = p - pr * OW;
            poff = pr * pm.sh * rg.pitch + pc * pm.sw;
        }
        const float* __restrict__ wrow = w + w_off(s, g, n, 0);
        uint32_t mine1 = kNoKey, mine2 = kNoKey;  // the results of the output this lane read
        auto step = [&](auto sub_c) __attribute__((always_inline)) {
            constexpr int sub = decltype(sub_c)::value;
            constexpr int ctrl = sub | (sub << 2) | (sub << 4) | (sub << 6);  // quad_perm [sub, sub, sub, sub]
            const int tt1 = __builtin_amdgcn_update_dpp(0, t1st, ctrl, 0xf, 0xf, true);
            const int po = __builtin_amdgcn_update_dpp(0, poff, ctrl, 0xf, 0xf, true);
            const float target1 = __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(val1), ctrl, 0xf, 0xf, true));
            int tt2 = -1;
            float target2 = 0.f;
            if constexpr (BOUND) {
                tt2 = __builtin_amdgcn_update_dpp(0, t2nd, ctrl, 0xf, 0xf, true);
                target2 = __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(val2), ctrl, 0xf, 0xf, true));
            }
            uint32_t key1 = kNoKey, key2 = kNoKey;
            // one walk over tile tt: the first output (distance, or lower bound) when `first`, the upper bound when
            // `second`
            auto walk = [&](int tt, bool first, bool second) __attribute__((always_inline)) {
#pragma unroll
                for (int h = KT / 16 - 1; h >= 0; h--) {  // descending: the lowest matching k is kept
                    const int k = tt * KT + (lane & 3) * 4 + 16 * h;
                    if (k < K) {
                        float wv[4];
                        if (w_vec) {
                            const float4 w4 = *reinterpret_cast<const float4*>(wrow + k);
                            wv[0] = w4.x; wv[1] = w4.y; wv[2] = w4.z; wv[3] = w4.w;
                        } else {
#pragma unroll
                            for (int j = 0; j < 4; j++) wv[j] = k + j < K ? wrow[k + j] : 0.f;
                        }
                        const int4 tp4 = *reinterpret_cast<const int4*>(tab + k);  // (k is a multiple of four)
                        const int tp[4] = {tp4.x, tp4.y, tp4.z, tp4.w};
                        float xa[4], xb[4];  // the reads leave together
#pragma unroll
                        for (int j = 0; j < 4; j++) {
                            xa[j] = xs[tp[j] + po];
                            xb[j] = BOUND ? xs[cg * E + tp[j] + po] : 0.f;
                        }
#pragma unroll
                        for (int j = 3; j >= 0; j--) {
                            if constexpr (!BOUND) {
                                const float d = xa[j] - wv[j];
                                if (fabsf(d) == target1 && k + j < K) key1 = ((uint32_t)(k + j) << 1) | (!(d >= 0) ? 1u : 0u);
                            } else {
                                const float t1 = wv[j] - xa[j], t2 = xb[j] - wv[j];
                                const uint32_t kk = ((uint32_t)(k + j) << 1) | (!(t1 <= t2) ? 1u : 0u);
                                if (first && fminf(t1, t2) == target1 && k + j < K) key1 = kk;
                                if (second && fmaxf(t1, t2) == target2 && k + j < K) key2 = kk;
                            }
                        }
                    }
                }
            };
            if (tt1 >= 0) walk(tt1, true, BOUND && tt2 == tt1);
            if constexpr (BOUND) {
                if (tt2 >= 0 && tt2 != tt1) walk(tt2, false, true);
            }
            // lowest key of the four lanes that share the output (all lanes of the wave are here)
            key1 = min(key1, (uint32_t)__builtin_amdgcn_update_dpp(0, (int)key1, 0xB1, 0xf, 0xf, true));   // quad_perm [1,0,3,2]
            key1 = min(key1, (uint32_t)__builtin_amdgcn_update_dpp(0, (int)key1, 0x4E, 0xf, 0xf, true));   // quad_perm [2,3,0,1]
            if ((lane & 3) == sub) mine1 = key1;
            if constexpr (BOUND) {
                key2 = min(key2, (uint32_t)__builtin_amdgcn_update_dpp(0, (int)key2, 0xB1, 0xf, 0xf, true));
                key2 = min(key2, (uint32_t)__builtin_amdgcn_update_dpp(0, (int)key2, 0x4E, 0xf, 0xf, true));
                if ((lane & 3) == sub) mine2 = key2;
            }
        };
        step(std::integral_constant<int, 0>{}); step(std::integral_constant<int, 1>{});
        step(std::integral_constant<int, 2>{}); step(std::integral_constant<int, 3>{});
        if (live) {
            uint32_t code = BOUND ? kNoGradId : 0u;  // a lower bound of zero has no arg-max
            if (t1st >= 0 && mine1 != kNoKey) code = (mine1 >> 1) | ((mine1 & 1u) ? kSignBit : 0u);
            pos1[o] = (int32_t)code;
            if constexpr (BOUND) {
                code = 0u;
                if (t2nd >= 0 && mine2 != kNoKey) code = (mine2 >> 1) | ((mine2 & 1u) ? kSignBit : 0u);
                pos2[o] = (int32_t)code;
            }
        }
    }
}

// Row blocks of the image kernels (second pass here, the gradient scatter of bwd_scatter.hip): `arrays` staged copies
// of the image rows under a block of output rows, plus the table of taps.  False when they do not fit.
inline bool image_row_blocks(const Geom& s, const PatchMap& pm, int arrays, ImageRowBlocks* out, size_t* lds_bytes) {
    const int OW = pm.OW, OH = OW > 0 ? s.HW / OW : 0, kh = pm.taps / pm.kw;
    if (OW <= 0 || OH * OW != s.HW || s.CIg > kRiMaxK) return false;
    ImageRowBlocks rg{};
    rg.R = OW >= 64 ? 1 : std::min(OH, std::max(1, 64 / OW));
    rg.rows_in = (rg.R - 1) * pm.sh + (kh - 1) * pm.dh + 1;
    rg.pitch = pm.W + 2 * pm.pw;
    const long e = (long)rg.rows_in * rg.pitch;
    if (e > 64 * kRiMaxSlots) return false;
    rg.E = (int)e;
    rg.nrb = ceil_div(OH, rg.R);
    rg.nt = 0;
    rg.inv_pitch = 1.0f / (float)rg.pitch;
    rg.inv_ow = 1.0f / (float)OW;
    const size_t lds = ((size_t)arrays * pm.cg * rg.E + (size_t)((s.CIg + 3) & ~3)) * sizeof(float);
    if (lds > (size_t)kRiLdsBudget) return false;
    if ((long)s.B * s.G * rg.nrb >= (1L << 31)) return false;
    *out = rg;
    *lds_bytes = lds;
    return true;
}

// tuning aid: NORM_DIST_RESCAN_IMAGE=0 keeps the sorted second pass for images too
inline bool rescan_image_enabled() {
    const char* v = getenv("NORM_DIST_RESCAN_IMAGE");  // read at every call: the tests switch it
    return v == nullptr || v[0] != '0';
}

// Launches the second pass on staged image rows; -1 when the geometry does not fit (the caller falls back on the
// sorted second pass).  BOUND: out1 / pos1 are the lower outputs, out2 / pos2 the upper ones.
template <bool BOUND>
int launch_rescan_image(const float* x, const float* x2, const float* w, const float* out1, int32_t* pos1,
                        const float* out2, int32_t* pos2, const Geom& s, int kt, hipStream_t st, const PatchMap& pm) {
    if (kt != 16 && kt != 32) return -1;
    ImageRowBlocks rg{};
    size_t lds = 0;
    if (!image_row_blocks(s, pm, BOUND ? 2 : 1, &rg, &lds)) return -1;
    rg.nt = ceil_div(s.CIg, kt);
    const long nwg = (long)s.B * s.G * rg.nrb;
    // two 512-thread workgroups per compute unit when their LDS allows it, else one of 1024 threads
    const int threads = 2 * lds <= (size_t)kRiLdsBudget ? 512 : 1024;
    const int w_vec = s.CIg % 4 == 0 && (uintptr_t)w % 16 == 0;
#define NDIST_RESCAN_IMAGE(KT_)                                                                                          \
    do {                                                                                                                 \
        NDIST_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void*>(&rescan_image_kernel<BOUND, KT_>),               \
                                          hipFuncAttributeMaxDynamicSharedMemorySize, kRiLdsBudget));                    \
        hipLaunchKernelGGL((rescan_image_kernel<BOUND, KT_>), dim3((unsigned)nwg), dim3(threads), lds, st, x, x2, w, out1, \
                           pos1, out2, pos2, s, pm, rg, w_vec);                                                          \
    } while (0)
    if (kt == 16) NDIST_RESCAN_IMAGE(16);
    else NDIST_RESCAN_IMAGE(32);
#undef NDIST_RESCAN_IMAGE
    return hip_failed(hipGetLastError()) ? 4 : 0;
}

}  // namespace ndist
