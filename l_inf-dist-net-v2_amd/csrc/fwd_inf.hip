// Forward of the infinity distance: out = max(1e-10, max_k |x - w|), optionally with the signed arg-max code.
// Replaces inf_dist::forward / inf_dist::forward_nograd of the reference (core/cuda/inf_dist_cuda.cu:14-198,248-317).
//
// Arg-max without per-pair bookkeeping: the main kernel only keeps, per output, the running maximum and the index
// of the last k-tile (32 consecutive k) that strictly raised it.  The first k attaining the final maximum lies in
// that tile (later tiles that merely equal it do not register), so a small second kernel rescans those 32 pairs,
// takes the lowest k whose |x - w| equals the maximum bit for bit, and writes the code (index, sign flag).  The
// subtraction is the same fp32 operation in both kernels, so the comparison is exact.  In the conv layout the
// second pass is the sorted rescan of rescan_sorted.h; the thread-per-output kernel below serves HW == 1 and
// very small HW.
#include "fwd_tile.h"
#include "rescan_sorted.h"
#include "rescan_image.h"

namespace ndist {

//
// BOUNDED: whole k-tiles are skipped (fully-connected layout, large problems).  A wave drops the 32 k of a step when
// max|x| + max|w| over those k (precomputed per row) cannot reach what each of its outputs already has: the running
// maximum, or before that the output's seed, an actual pair of the reduction found by a pre-pass (see launch_seeds).
// Values: a skipped tile holds nothing above the final maximum.  Arg-max: a tile is skipped only when its bound is
// BELOW the seed (strictly), or at or below the running maximum of the tiles already seen, which all have lower k;
// either way it cannot hold the first occurrence of the final maximum, so the recorded tile is the same one.
template <bool TRACK, bool BOUNDED = false>
struct OpInf {
    static constexpr int NX = 1, PHASES = 1, NOF = 1, NOI = TRACK ? 1 : 0;
    static constexpr bool PREFETCH = !TRACK;
    static constexpr bool PREFETCH_SMALL = true;
    static constexpr bool HEAVY = TRACK;
    static constexpr bool TILE_BOUND = BOUNDED;
    static constexpr float COST = TRACK ? 6.2f : 5.2f;  // issue cycles per pair and wave (launcher's cost model)
    struct AccPlain { float m; };
    struct AccTrack { float m; float prev; int cid; };
    using Acc = typename std::conditional<TRACK, AccTrack, AccPlain>::type;

    __device__ static __forceinline__ void init(Acc& a, const FwdParams& P, int, int m, int n, int g) {
        a.m = kEps;
        if constexpr (TRACK) { a.prev = kEps; a.cid = -1; }
        if constexpr (BOUNDED) {
            // (fully-connected layout: row m, column n of group g)
            if (m < P.s.M && n < P.s.COg) {
                const float seed = P.aux != nullptr ? P.aux[y_off(P.s, m, g, n, 0)] : kEps;
                if constexpr (TRACK) {
                    // `prev` doubles as the skip threshold: the float just below the seed, so that the tile of the
                    // seed's pair (bound >= seed) is looked at and registers as the first to reach its value
                    a.prev = fmaxf(kEps, __uint_as_float(__float_as_uint(seed) - 1u));
                } else {
                    a.m = fmaxf(kEps, seed);  // the seed is a pair of the reduction: the maximum may start there
                }
            } else {  // padding of the tile, never stored: everything can be skipped
                if constexpr (TRACK) a.prev = __builtin_inff();
                else a.m = __builtin_inff();
            }
        }
    }
    template <int TM, int TN>
    __device__ static __forceinline__ bool tile_skip(const Acc (&a)[TM][TN], const float (&bx)[TM], const float (&bw)[TN]) {
        bool hot = false;
#pragma unroll
        for (int i = 0; i < TM; i++)
#pragma unroll
            for (int j = 0; j < TN; j++) {
                if constexpr (TRACK) hot |= bx[i] + bw[j] > a[i][j].prev;
                else hot |= bx[i] + bw[j] > a[i][j].m;
            }
        return __builtin_amdgcn_ballot_w64(hot) == 0;
    }
    template <int TN>
    __device__ static __forceinline__ void row2(Acc (&a)[TN], const FwdParams&, int, float x0, float, const float (&w0)[TN],
                                                float x1, float, const float (&w1)[TN]) {
        // two subtractions feeding one three-operand maximum, pair by pair: the maximum runs in the slower of the
        // two vector pipes and overlaps best with subtractions right next to it
#pragma unroll
        for (int j = 0; j < TN; j++) {
            const float d0 = x0 - w0[j], d1 = x1 - w1[j];
            a[j].m = fmaxf(fmaxf(a[j].m, fabsf(d0)), fabsf(d1));
        }
    }
    __device__ static __forceinline__ void phase_end(Acc& a, const FwdParams&, int, int tile) {
        if constexpr (TRACK) {
            // the maximum never falls, so the previous value is refreshed with a plain move (with a seed the running
            // maximum may still be below the threshold the seed left in prev)
            a.cid = a.m > a.prev ? tile : a.cid;
            a.prev = BOUNDED ? fmaxf(a.prev, a.m) : a.m;
        }
    }
    __device__ static __forceinline__ void merge(Acc& a, const Acc& b, const FwdParams&) {
        if constexpr (TRACK) {
            // equal maxima: the earlier tile holds the first occurrence; -1 (nothing found) never wins a tie
            if (b.m > a.m || (b.m == a.m && (unsigned)b.cid < (unsigned)a.cid)) { a.m = b.m; a.cid = b.cid; }
        } else {
            a.m = fmaxf(a.m, b.m);
        }
    }
    __device__ static __forceinline__ void finalize(const Acc& a, const FwdParams&, float* fv, int* iv) {
        fv[0] = a.m;
        if constexpr (TRACK) iv[0] = a.cid;
    }
};

// pos holds the winning k-tile per output on entry and the arg-max code on exit.
// implicit != 0: x holds images and pm maps the unfolded coordinates to them (vec is 0 then).
template <int KT>
__global__ __launch_bounds__(256) void inf_rescan_kernel(const float* __restrict__ x, const float* __restrict__ w,
                                                         const float* __restrict__ out, int32_t* __restrict__ pos,
                                                         const Geom s, long total, int vec, int implicit,
                                                         const PatchMap pm, const int* __restrict__ gate) {
    constexpr int kt = KT;
    const long o = (long)blockIdx.x * 256 + threadIdx.x;
    if (o >= total || (gate != nullptr && gate[0] >= 1)) return;
    const int cid = pos[o];
    if (cid < 0) {  // nothing exceeded the floor
        pos[o] = 0;
        return;
    }
    const int hw = (int)(o % s.HW);
    const long r = o / s.HW;
    const int gco = (int)(r % (s.COg * s.G));
    const int b = (int)(r / (s.COg * s.G));
    const int g = gco / s.COg, co = gco - g * s.COg;
    const float val = out[o];
    const int k0 = cid * kt, k1 = min(k0 + kt, s.CIg);
    const float* __restrict__ xp = implicit ? x : x + x_off(s, b, g, 0, hw);
    const float* __restrict__ wp = w + w_off(s, g, co, 0);
    uint32_t code = 0;
    if (vec && k1 - k0 == kt) {
#pragma unroll
        for (int q = kt / 4 - 1; q >= 0; q--) {
            const float4 a = *reinterpret_cast<const float4*>(xp + k0 + 4 * q);
            const float4 c = *reinterpret_cast<const float4*>(wp + k0 + 4 * q);
            const float d[4] = {a.x - c.x, a.y - c.y, a.z - c.z, a.w - c.w};
#pragma unroll
            for (int j = 3; j >= 0; j--)
                if (fabsf(d[j]) == val) code = (uint32_t)(k0 + 4 * q + j) | (d[j] >= 0 ? 0u : kSignBit);
        }
    } else {
        for (int k = k1 - 1; k >= k0; k--) {  // descending: the lowest matching k is written last
            const float xv = implicit ? patch_elem(xp, pm, b, patch_tap(pm, g, k), hw) : xp[(long)k * s.HW];
            const float d = xv - wp[k];
            if (fabsf(d) == val) code = (uint32_t)k | (d >= 0 ? 0u : kSignBit);
        }
    }
    pos[o] = (int32_t)code;
}

// Problems below the size of the seeded kernels on which the hot-tile path is still tried first (its pre-pass reads
// all of x and w once, so it pays from about this many pairs on); the plain kernels stay queued behind it, gated.
bool hot_alone_applies(const Geom& s) {
    const double pairs = (double)s.M * s.COg * s.G * s.CIg;
    return s.HW == 1 && !skinny_applies(s) && skip_override_limit(1) > 0 && pairs >= 5e7 && s.M >= 8;
}

bool seeded_forward_applies(const Geom& s) {
    const double pairs = (double)s.M * s.COg * s.G * s.CIg;
    return s.HW == 1 && !skinny_applies(s) && skip_override_limit(1) > 0 &&
           ((pairs >= 2e8 && s.M >= kMinSeededRows) || skip_forced_on());
}

int launch_inf_forward(const float* x, const float* w, const Geom& s, float* out, int32_t* pos, hipStream_t st,
                       const UnfoldGeom* cv, const WeightSeeds* wpre, const SharedFront* front) {
    FwdParams P{};
    P.x = x;
    P.w = w;
    P.out = out;
    P.pos = pos;
    P.s = s;
    PatchMap pm{};
    if (cv != nullptr) {
        pm = make_patch_map(*cv, s.G);
        P.implicit = 1;
        P.pm = pm;
    }
    // Large fully-connected problems: seeds and k-tile bounds from three small pre-pass kernels, then the operator
    // that skips the k-tiles which cannot matter (most of them, unless the largest |x - w| are far below
    // max|x| + max|w| everywhere).  NORM_DIST_SKIP=0 / ndist_set_skip_mode(0, ..) switches this off, 1 forces it on
    // for small problems too.
    // Before those: from the same row pre-pass the hot-tile kernels (fwd_hot.hip) find out on the device whether
    // few k-tiles decide all maxima; if so they produce the outputs themselves and everything queued below is gated off.
    const bool bounded = cv == nullptr && seeded_forward_applies(s);
    const bool hot = cv == nullptr && hot_forward_applies(s) && (bounded || hot_alone_applies(s));
    float* scratch = nullptr;
    const int* gate = nullptr;
    KernelTimer timer(st);  // pre-passes + tiled kernel + rescan
    if (bounded || hot) {
        const size_t nseed = seed_scratch_floats(s);
        SeedBuffers sb{};
        int rs = 0;
        if (front != nullptr) {
            scratch = front->scratch;
            sb = front->sb;
        } else {
            NDIST_HIP_TRY(scratch_alloc((void**)&scratch, (nseed + (hot ? hot_scratch_floats(s) : 0)) * sizeof(float), st));
            rs = launch_row_seeds(x, w, s, scratch, nullptr, 0, st, &sb, nullptr, wpre,
                                  hot ? reinterpret_cast<int*>(scratch + nseed) : nullptr);
        }
        // (with the hot-tile kernels ahead, their second launch computes the output seeds when the plan says no)
        if (!rs && hot)
            rs = launch_inf_hot(x, w, s, sb, scratch + nseed, out, pos, st, &gate, bounded, front != nullptr && front->plan_done);
        if (!rs && bounded && !hot) rs = launch_output_seeds(x, w, s, sb, gate, 1, st);
        if (rs) {
            if (front == nullptr) (void)scratch_free(scratch, st);
            return rs;
        }
        if (gate != nullptr) {
            P.gate = gate;
            P.gate_limit = 1;
            P.gate_sense = 1;
        }
        if (bounded) {
            P.aux = sb.seed;
            P.tile_x = sb.tile_x;
            P.tile_w = sb.tile_w;
            P.ntile32 = sb.ntile;
        }
    }
    // (the scratch holds the gate: it is released after the last kernel that reads it has been queued)
    auto done = [&](int rc) {
        if ((bounded || hot) && front == nullptr && hip_failed(scratch_free(scratch, st)) && !rc) rc = 4;
        return rc;
    };
    // With the hot-tile plan ahead there are two dense candidates behind it: the kernel that drops k-tiles by their
    // bounds, and, for data on which the plan found (nearly) every tile hot, the plain kernel (gate words 4 and 5 of
    // the plan's decision; both leave the winning k-tile in pos, in the same configuration).
    const bool two = bounded && hot && gate != nullptr;
    FwdParams Q = P;  // the plain candidate
    if (two) {
        P.gate = gate + 4;
        Q.gate = gate + 5;
        Q.aux = nullptr;
        Q.tile_x = Q.tile_w = nullptr;
    }
    if (pos == nullptr) {
        int rc = bounded ? launch_fwd<OpInf<false, true>, CfgWideT, CfgMid, CfgSmall>(P, st)
                         : launch_fwd_conv<OpInf<false>, CfgWide4, CfgBig, CfgSmall, CfgWide>(P, st);
        if (!rc && two) rc = launch_fwd_conv<OpInf<false>, CfgWide4, CfgBig, CfgSmall, CfgWide>(Q, st);
        return done(rc);
    }
    int kt = 0;
    int rc = bounded ? launch_fwd_layouts<false, OpInf<true, true>, CfgWideT, CfgMid, CfgSmall>(P, st, &kt)
                     : launch_fwd_layouts<true, OpInf<true>, CfgWideT, CfgMid, CfgSmall4>(P, st, &kt);
    if (!rc && two) {
        int kt2 = 0;
        rc = launch_fwd_layouts<true, OpInf<true>, CfgWideT, CfgMid, CfgSmall4>(Q, st, &kt2);
        if (!rc && kt2 != kt) rc = 2;  // (same candidate list and cost model: cannot differ)
    }
    if (rc) return done(rc);
    if (cv != nullptr && rescan_image_enabled()) {  // images: the second pass on staged image rows, where they fit
        const int r = launch_rescan_image<false>(x, nullptr, w, out, pos, nullptr, nullptr, s, kt, st, pm);
        if (r != -1) return done(r);
    }
    if (rescan_sorted_applies(s, kt))
        return done(launch_rescan_sorted<0>(x, nullptr, w, out, pos, s, kt, st, cv ? &pm : nullptr));
    const long total = (long)s.M * s.COg * s.G;
    const int imp = cv != nullptr;
    const int vec = !imp && s.HW == 1 && s.CIg % 4 == 0 && (uintptr_t)x % 16 == 0 && (uintptr_t)w % 16 == 0;
    const dim3 grid((unsigned)((total + 255) / 256));
#define NDIST_INF_RESCAN(KT_) \
    hipLaunchKernelGGL(inf_rescan_kernel<KT_>, grid, dim3(256), 0, st, x, w, out, pos, s, total, vec, imp, pm, gate)
    if (kt == 4) NDIST_INF_RESCAN(4);
    else if (kt == 16) NDIST_INF_RESCAN(16);
    else if (kt == 32) NDIST_INF_RESCAN(32);
    else return done(2);
#undef NDIST_INF_RESCAN
    return done(hip_failed(hipGetLastError()) ? 4 : 0);
}

}  // namespace ndist
