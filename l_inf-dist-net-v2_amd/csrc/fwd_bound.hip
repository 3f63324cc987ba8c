// Forward of the interval bounds of the infinity distance over an input box [xL, xU]:
//   t1 = w - xL, t2 = xU - w;  yL = -min(-1e-10, min_k min(t1, t2));  yU = max(1e-10, max_k max(t1, t2))
// optionally with the two arg-max codes.  Replaces bound_inf_dist::forward / forward_nograd of the reference
// (core/cuda/bound_inf_dist_cuda.cu:15-238,304-345).  Arg-max by k-tile bookkeeping plus a rescan kernel, as in the
// infinity-distance forward.
#include <type_traits>

#include "fwd_tile.h"
#include "rescan_sorted.h"
#include "rescan_image.h"

namespace ndist {

// BOUNDED: whole k-tiles are skipped, as in the infinity-distance forward.  Both candidates of a pair lie within
// +-(max(|xL|, |xU|) + max|w|) over the tile; when that bound reaches neither what the upper reduction nor (negated)
// what the lower reduction of any output of the wave already has, the tile cannot change them.  Both start from
// seeds, actual pairs found by a pre-pass (see launch_seeds).  With arg-max the thresholds are the bookkeeping
// registers plo / phi, started one float inside the seeds: a tile is skipped only when it is strictly short of the
// seed, or does not pass the running extremes of the tiles before it, so it never holds the first k that attains
// a final extreme, and the recorded tiles are those of the plain kernel.
template <bool TRACK, bool BOUNDED = false>
struct OpBound {
    static constexpr int NX = 2, PHASES = 1, NOF = 2, NOI = TRACK ? 2 : 0;
    static constexpr bool PREFETCH = false;  // two x arrays: the operand set is already large
    static constexpr bool PREFETCH_SMALL = true;
    static constexpr bool HEAVY = true;
    static constexpr bool TILE_BOUND = BOUNDED;
    static constexpr float COST = TRACK ? 18.f : 15.f;  // issue cycles per pair and wave (launcher's cost model)
    struct AccPlain { float lo, hi; };
    struct AccTrack { float lo, hi, plo, phi; int clo, chi; };
    using Acc = typename std::conditional<TRACK, AccTrack, AccPlain>::type;

    __device__ static __forceinline__ void init(Acc& a, const FwdParams& P, int, int m, int n, int g) {
        a.lo = -kEps;
        a.hi = kEps;
        if constexpr (TRACK) { a.plo = -kEps; a.phi = kEps; a.clo = -1; a.chi = -1; }
        if constexpr (BOUNDED) {
            if (m < P.s.M && n < P.s.COg) {  // (fully-connected layout: row m, column n of group g)
                if (P.aux != nullptr) {
                    const float sh = P.aux[y_off(P.s, m, g, n, 0)], sl = P.aux2[y_off(P.s, m, g, n, 0)];
                    if constexpr (TRACK) {
                        // the floats just inside the seeds (sh >= 1e-10 > 0 > -1e-10 >= sl: one step towards zero)
                        a.phi = fmaxf(kEps, __uint_as_float(__float_as_uint(sh) - 1u));
                        a.plo = fminf(-kEps, __uint_as_float(__float_as_uint(sl) - 1u));
                    } else {
                        a.hi = fmaxf(kEps, sh);
                        a.lo = fminf(-kEps, sl);
                    }
                }
            } else {  // padding of the tile, never stored: everything can be skipped
                if constexpr (TRACK) {
                    a.phi = __builtin_inff();
                    a.plo = -__builtin_inff();
                } else {
                    a.hi = __builtin_inff();
                    a.lo = -__builtin_inff();
                }
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
                const float b = bx[i] + bw[j];
                if constexpr (TRACK) hot |= b > a[i][j].phi || b > -a[i][j].plo;
                else hot |= b > a[i][j].hi || b > -a[i][j].lo;
            }
        return __builtin_amdgcn_ballot_w64(hot) == 0;
    }
    template <int TN>
    __device__ static __forceinline__ void row2(Acc (&a)[TN], const FwdParams&, int, float l0, float u0, const float (&w0)[TN],
                                                float l1, float u1, const float (&w1)[TN]) {
        // column by column: the four subtractions of a column next to its min3 / max3 pair (the two kinds of
        // instruction issue to different pipes and overlap best when they alternate)
#pragma unroll
        for (int j = 0; j < TN; j++) {
            const float s1 = w0[j] - l0, s2 = u0 - w0[j], t1 = w1[j] - l1, t2 = u1 - w1[j];
            a[j].lo = fminf(fminf(a[j].lo, s1), s2);
            a[j].hi = fmaxf(fmaxf(a[j].hi, s1), s2);
            a[j].lo = fminf(fminf(a[j].lo, t1), t2);
            a[j].hi = fmaxf(fmaxf(a[j].hi, t1), t2);
        }
    }
    __device__ static __forceinline__ void phase_end(Acc& a, const FwdParams&, int, int tile) {
        if constexpr (TRACK) {
            if (a.lo < a.plo) { a.clo = tile; a.plo = a.lo; }
            if (a.hi > a.phi) { a.chi = tile; a.phi = a.hi; }
        }
    }
    __device__ static __forceinline__ void merge(Acc& a, const Acc& b, const FwdParams&) {
        if constexpr (TRACK) {
            if (b.lo < a.lo || (b.lo == a.lo && (unsigned)b.clo < (unsigned)a.clo)) { a.lo = b.lo; a.clo = b.clo; }
            if (b.hi > a.hi || (b.hi == a.hi && (unsigned)b.chi < (unsigned)a.chi)) { a.hi = b.hi; a.chi = b.chi; }
        } else {
            a.lo = fminf(a.lo, b.lo);
            a.hi = fmaxf(a.hi, b.hi);
        }
    }
    __device__ static __forceinline__ void finalize(const Acc& a, const FwdParams&, float* fv, int* iv) {
        fv[0] = -a.lo;
        fv[1] = a.hi;
        if constexpr (TRACK) { iv[0] = a.clo; iv[1] = a.chi; }
    }
};

// posL / posU hold the winning k-tiles on entry and the arg-max codes on exit
// (lower bound untouched by any k: the "no gradient" code 0xffffffff; upper bound untouched: 0).
template <int KT>
__global__ __launch_bounds__(256) void bound_rescan_kernel(const float* __restrict__ xl, const float* __restrict__ xu,
                                                           const float* __restrict__ w, const float* __restrict__ yl,
                                                           const float* __restrict__ yu, int32_t* __restrict__ posl,
                                                           int32_t* __restrict__ posu, const Geom s, long total, int vec,
                                                           int implicit, const PatchMap pm,
                                                           const int* __restrict__ gate) {
    const long o = (long)blockIdx.x * 256 + threadIdx.x;
    if (o >= total || (gate != nullptr && gate[0] >= 1)) return;
    const int hw = (int)(o % s.HW);
    const long r = o / s.HW;
    const int gco = (int)(r % (s.COg * s.G));
    const int b = (int)(r / (s.COg * s.G));
    const int g = gco / s.COg, co = gco - g * s.COg;
    // implicit != 0: xl / xu hold images and pm maps the unfolded coordinates to them (vec is 0 then)
    const float* __restrict__ lp = implicit ? xl : xl + x_off(s, b, g, 0, hw);
    const float* __restrict__ up = implicit ? xu : xu + x_off(s, b, g, 0, hw);
    const float* __restrict__ wp = w + w_off(s, g, co, 0);
    // one k of the tile: code when the pair attains the target (descending scans keep the lowest k)
    auto probe = [&](bool upper, float a, float c, float wv, float target, int k, uint32_t& code) {
        if (a > c) a = c = (a + c) * 0.5f;
        const float t1 = wv - a, t2 = c - wv;
        const float e = upper ? fmaxf(t1, t2) : fminf(t1, t2);
        if (e == target) code = (uint32_t)k | (t1 <= t2 ? 0u : kSignBit);
    };
    auto scan = [&](bool upper, int tile, float target, uint32_t code) -> uint32_t {
        const int k0 = tile * KT, k1 = min(k0 + KT, s.CIg);
        if (vec && k1 - k0 == KT) {
#pragma unroll
            for (int q = KT / 4 - 1; q >= 0; q--) {
                const float4 a = *reinterpret_cast<const float4*>(lp + k0 + 4 * q);
                const float4 c = *reinterpret_cast<const float4*>(up + k0 + 4 * q);
                const float4 v = *reinterpret_cast<const float4*>(wp + k0 + 4 * q);
                probe(upper, a.w, c.w, v.w, target, k0 + 4 * q + 3, code);
                probe(upper, a.z, c.z, v.z, target, k0 + 4 * q + 2, code);
                probe(upper, a.y, c.y, v.y, target, k0 + 4 * q + 1, code);
                probe(upper, a.x, c.x, v.x, target, k0 + 4 * q + 0, code);
            }
        } else {
            for (int k = k1 - 1; k >= k0; k--) {
                if (implicit) {
                    const PatchTap tp = patch_tap(pm, g, k);
                    probe(upper, patch_elem(lp, pm, b, tp, hw), patch_elem(up, pm, b, tp, hw), wp[k], target, k, code);
                } else {
                    probe(upper, lp[(long)k * s.HW], up[(long)k * s.HW], wp[k], target, k, code);
                }
            }
        }
        return code;
    };
    const int cl = posl[o], cu = posu[o];
    uint32_t codel = kNoGradId, codeu = 0;
    if (cl >= 0) codel = scan(false, cl, -yl[o], codel);
    if (cu >= 0) codeu = scan(true, cu, yu[o], codeu);
    posl[o] = (int32_t)codel;
    posu[o] = (int32_t)codeu;
}

int launch_bound_forward(const float* xl, const float* xu, const float* w, const Geom& s, float* yl, float* yu,
                         int32_t* pl, int32_t* pu, hipStream_t st, const UnfoldGeom* cv, const WeightSeeds* wpre,
                         const SharedFront* front) {
    FwdParams P{};
    PatchMap pm{};
    if (cv != nullptr) {
        pm = make_patch_map(*cv, s.G);
        P.implicit = 1;
        P.pm = pm;
    }
    P.x = xl;
    P.x2 = xu;
    P.w = w;
    P.out = yl;
    P.out2 = yu;
    P.pos = pl;
    P.pos2 = pu;
    P.s = s;
    // large fully-connected problems: hot-tile kernels first, else seeds and k-tile bounds, as in launch_inf_forward
    const bool bounded = cv == nullptr && seeded_forward_applies(s);
    const bool hot = cv == nullptr && hot_forward_applies(s) && (bounded || hot_alone_applies(s));
    if (!bounded && !hot && pl == nullptr) return launch_fwd_conv<OpBound<false>, CfgBoundN, CfgSmall>(P, st);
    KernelTimer timer(st);  // pre-passes + tiled kernel + rescan
    float* scratch = nullptr;
    const int* gate = nullptr;
    if (bounded || hot) {
        const size_t nseed = bound_seed_scratch_floats(s);
        SeedBuffers sb{};
        int rs = 0;
        if (front != nullptr) {
            scratch = front->scratch;
            sb = front->sb;
        } else {
            NDIST_HIP_TRY(scratch_alloc((void**)&scratch, (nseed + (hot ? hot_scratch_floats(s) : 0)) * sizeof(float), st));
            rs = launch_row_seeds(xl, w, s, scratch, nullptr, 0, st, &sb, xu, wpre,
                                  hot ? reinterpret_cast<int*>(scratch + nseed) : nullptr);
        }
        if (!rs && hot)
            rs = launch_bound_hot(xl, xu, w, s, sb, scratch + nseed, yl, yu, pl, pu, st, &gate, bounded,
                                  front != nullptr && front->plan_done);
        if (!rs && bounded && !hot) rs = launch_output_seeds(xl, w, s, sb, gate, 1, st, xu);
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
            P.aux2 = sb.seed2;
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
    // two dense candidates behind the hot-tile plan, as in launch_inf_forward
    const bool two = bounded && hot && gate != nullptr;
    FwdParams Q = P;  // the plain candidate
    if (two) {
        P.gate = gate + 4;
        Q.gate = gate + 5;
        Q.aux = Q.aux2 = nullptr;
        Q.tile_x = Q.tile_w = nullptr;
    }
    if (pl == nullptr) {
        int rc = bounded ? launch_fwd<OpBound<false, true>, CfgBoundT, CfgMid, CfgSmall>(P, st)
                         : launch_fwd_conv<OpBound<false>, CfgBoundN, CfgSmall>(P, st);
        if (!rc && two) rc = launch_fwd_conv<OpBound<false>, CfgBoundN, CfgSmall>(Q, st);
        return done(rc);
    }
    int kt = 0;
    int rc = bounded ? launch_fwd_layouts<false, OpBound<true, true>, CfgBoundT, CfgSmall>(P, st, &kt)
                     : launch_fwd_layouts<true, OpBound<true>, CfgBoundT, CfgSmall>(P, st, &kt);
    if (!rc && two) {
        int kt2 = 0;
        rc = launch_fwd_layouts<true, OpBound<true>, CfgBoundT, CfgSmall>(Q, st, &kt2);
        if (!rc && kt2 != kt) rc = 2;  // (same candidate list and cost model: cannot differ)
    }
    if (rc) return done(rc);
    const int imp = cv != nullptr;
    if (imp && rescan_image_enabled()) {  // images: both second passes on one staged pair of image rows
        const int r = launch_rescan_image<true>(xl, xu, w, yl, pl, yu, pu, s, kt, st, pm);
        if (r != -1) return done(r);
    }
    if (rescan_sorted_applies(s, kt)) {
        const int r1 = launch_rescan_sorted<1>(xl, xu, w, yl, pl, s, kt, st, imp ? &pm : nullptr);
        return done(r1 ? r1 : launch_rescan_sorted<2>(xl, xu, w, yu, pu, s, kt, st, imp ? &pm : nullptr));
    }
    const long total = (long)s.M * s.COg * s.G;
    const int vec = !imp && s.HW == 1 && s.CIg % 4 == 0 && (uintptr_t)xl % 16 == 0 && (uintptr_t)xu % 16 == 0 &&
                    (uintptr_t)w % 16 == 0;
    const dim3 grid((unsigned)((total + 255) / 256));
#define NDIST_BOUND_RESCAN(KT_) \
    hipLaunchKernelGGL(bound_rescan_kernel<KT_>, grid, dim3(256), 0, st, xl, xu, w, yl, yu, pl, pu, s, total, vec, imp, pm, gate)
    if (kt == 4) NDIST_BOUND_RESCAN(4);
    else if (kt == 16) NDIST_BOUND_RESCAN(16);
    else if (kt == 32) NDIST_BOUND_RESCAN(32);
    else return done(2);
#undef NDIST_BOUND_RESCAN
    return done(hip_failed(hipGetLastError()) ? 4 : 0);
}

// A layer's distance and its interval bounds in one call (certification runs both on every layer with the same
// weights, reference: core/modules/norm_dist.py:30-34): on problems large enough for the k-tile skipping variants the
// pre-pass over w (the largest of the pre-passes: it reads all of w) runs once and serves both operators.
int launch_inf_bound_forward(const float* x, const float* xl, const float* xu, const float* w, const Geom& s, float* out,
                             int32_t* pos, float* yl, float* yu, int32_t* pl, int32_t* pu, hipStream_t st,
                             const WeightSeeds* cached) {
    const bool bounded = seeded_forward_applies(s);
    const bool hot = hot_forward_applies(s) && (bounded || hot_alone_applies(s));
    if (!bounded && !hot) {
        const int rc = launch_inf_forward(x, w, s, out, pos, st);
        return rc ? rc : launch_bound_forward(xl, xu, w, s, yl, yu, pl, pu, st);
    }
    // One row pre-pass for x, the box and (unless the caller keeps them between calls) the weights, one launch of
    // the hot-tile plan for both operators; each operator's launcher goes on from there with its own scratch.
    const size_t na = seed_scratch_floats(s), nb = bound_seed_scratch_floats(s);
    const size_t nh = hot ? hot_scratch_floats(s) : 0;
    // (both blocks start on a multiple of four floats: the row pre-pass clears four ints at the head of the hot parts)
    const size_t sa = (na + nh + 3) / 4 * 4, sbz = nb + nh;
    float* block = nullptr;
    NDIST_HIP_TRY(scratch_alloc((void**)&block, (sa + sbz) * sizeof(float), st));
    SharedFront fa{block, SeedBuffers{}, hot}, fb{block + sa, SeedBuffers{}, hot};
    int rc = launch_joint_row_seeds(x, xl, xu, w, s, fa.scratch, fb.scratch, cached, st, &fa.sb, &fb.sb,
                                    hot ? reinterpret_cast<int*>(fa.scratch + na) : nullptr,
                                    hot ? reinterpret_cast<int*>(fb.scratch + nb) : nullptr);
    if (!rc && hot) rc = launch_joint_hot_plan(s, fa.sb, fa.scratch + na, fb.sb, fb.scratch + nb, st);
    const WeightSeeds shared{fa.sb.seed_w, fa.sb.seed_wk, fa.sb.tile_w};
    if (!rc) rc = launch_inf_forward(x, w, s, out, pos, st, nullptr, &shared, &fa);
    if (!rc) rc = launch_bound_forward(xl, xu, w, s, yl, yu, pl, pu, st, nullptr, &shared, &fb);
    if (hip_failed(scratch_free(block, st)) && !rc) rc = 4;
    return rc;
}

}  // namespace ndist
