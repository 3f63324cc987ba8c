// Operator policies of the finite-p forward for the tiled kernel skeleton (fwd_tile.h): the plain sum with |t|^p by
// repeated multiplication or through exp2/log2, the sum normalised by a running maximum for large p, and its
// pair-skipping variant.  Reference: core/cuda/norm_dist_cuda.cu:35-236,511-564, core/cuda/fast_pow.cuh:1-23.
#pragma once
#include "fwd_tile.h"

namespace ndist {

// |d|^IP = lo * hi for IP in 1..10, where lo = |d| (odd IP) or the running even power; this computes, in place and in
// stages over all N values (neighbouring instructions independent), d <- lo and hi, so that the caller finishes
// with one fused multiply-add per value.  For even IP the returned lo is an even power and needs no absolute value.
template <int IP, int N>
__device__ __forceinline__ void abs_pow_split(float (&d)[N], float (&hi)[N]) {
    static_assert(IP >= 1 && IP <= 10, "ladder range");
    if constexpr (IP == 1) {
#pragma unroll
        for (int j = 0; j < N; j++) hi[j] = 1.0f;
    } else if constexpr (IP == 2) {
#pragma unroll
        for (int j = 0; j < N; j++) hi[j] = d[j];
    } else if constexpr (IP == 3) {
#pragma unroll
        for (int j = 0; j < N; j++) hi[j] = d[j] * d[j];
    } else if constexpr (IP == 4) {
#pragma unroll
        for (int j = 0; j < N; j++) { d[j] = d[j] * d[j]; hi[j] = d[j]; }
    } else if constexpr (IP == 5) {
#pragma unroll
        for (int j = 0; j < N; j++) hi[j] = d[j] * d[j];
#pragma unroll
        for (int j = 0; j < N; j++) hi[j] = hi[j] * hi[j];
    } else if constexpr (IP == 6) {
#pragma unroll
        for (int j = 0; j < N; j++) d[j] = d[j] * d[j];
#pragma unroll
        for (int j = 0; j < N; j++) hi[j] = d[j] * d[j];
    } else if constexpr (IP == 7) {
#pragma unroll
        for (int j = 0; j < N; j++) hi[j] = d[j] * d[j];
        float t[N];
#pragma unroll
        for (int j = 0; j < N; j++) t[j] = hi[j] * hi[j];
#pragma unroll
        for (int j = 0; j < N; j++) hi[j] = t[j] * hi[j];
    } else if constexpr (IP == 8) {
#pragma unroll
        for (int j = 0; j < N; j++) d[j] = d[j] * d[j];
#pragma unroll
        for (int j = 0; j < N; j++) { d[j] = d[j] * d[j]; hi[j] = d[j]; }
    } else if constexpr (IP == 9) {
#pragma unroll
        for (int j = 0; j < N; j++) hi[j] = d[j] * d[j];
#pragma unroll
        for (int j = 0; j < N; j++) hi[j] = hi[j] * hi[j];
#pragma unroll
        for (int j = 0; j < N; j++) hi[j] = hi[j] * hi[j];
    } else {
        float t[N];
#pragma unroll
        for (int j = 0; j < N; j++) d[j] = d[j] * d[j];
#pragma unroll
        for (int j = 0; j < N; j++) t[j] = d[j] * d[j];
#pragma unroll
        for (int j = 0; j < N; j++) hi[j] = t[j] * t[j];
    }
}

__device__ __forceinline__ float root_p(float s, const FwdParams& P) { return fast_exp2(fast_log2(s) * P.inv_p); }

template <int IP>  // IP = 0: general p through exp2/log2
struct OpSum {
    static constexpr int NX = 1, PHASES = 1, NOF = 1, NOI = 0;
    static constexpr bool PREFETCH = true;
    static constexpr float COST = IP > 0 ? 10.5f : 25.8f;  // issue cycles per pair and wave (launcher's cost model)
    struct Acc { float s; };
    __device__ static __forceinline__ void init(Acc& a, const FwdParams&, int, int, int, int) { a.s = 0.f; }
    template <int TN>
    __device__ static __forceinline__ void row2(Acc (&a)[TN], const FwdParams& P, int, float x0, float, const float (&w0)[TN],
                                                float x1, float, const float (&w1)[TN]) {
        constexpr int N = 2 * TN;
        float d[N];
#pragma unroll
        for (int j = 0; j < TN; j++) { d[j] = x0 - w0[j]; d[TN + j] = x1 - w1[j]; }
        if constexpr (IP > 0) {
            float hi[N];  // |d|^IP = lo * hi with lo = |d| or d*d..., staged so that neighbours are independent
            abs_pow_split<IP, N>(d, hi);
#pragma unroll
            for (int j = 0; j < TN; j++) a[j].s = fmaf(IP & 1 ? fabsf(d[j]) : d[j], hi[j], a[j].s);
#pragma unroll
            for (int j = 0; j < TN; j++) a[j].s = fmaf(IP & 1 ? fabsf(d[TN + j]) : d[TN + j], hi[TN + j], a[j].s);
        } else {
            float e[N];
#pragma unroll
            for (int j = 0; j < N; j++) e[j] = fast_log2(fabsf(d[j]));
#pragma unroll
            for (int j = 0; j < N; j++) e[j] = fast_exp2(P.p * e[j]);
#pragma unroll
            for (int j = 0; j < TN; j++) a[j].s += e[j];
#pragma unroll
            for (int j = 0; j < TN; j++) a[j].s += e[TN + j];
        }
    }
    __device__ static __forceinline__ void phase_end(Acc&, const FwdParams&, int, int) {}
    __device__ static __forceinline__ void merge(Acc& a, const Acc& b, const FwdParams&) { a.s += b.s; }
    __device__ static __forceinline__ void finalize(const Acc& a, const FwdParams& P, float* fv, int*) {
        const float s = fmaxf(a.s, kFltMin);
        if constexpr (IP == 1) fv[0] = s;
        else if constexpr (IP == 2) fv[0] = sqrtf(s);
        else if constexpr (IP == 4) fv[0] = sqrtf(sqrtf(s));
        else if constexpr (IP == 8) fv[0] = sqrtf(sqrtf(sqrtf(s)));
        else fv[0] = root_p(s, P);
    }
};

// c = p * log2(m), rounded once.  The product must not be contracted into a later subtraction: c_old - p * log2(m)
// as one fused operation leaves the rounding residual of c_old instead of exactly 0 when m is unchanged, and the sum
// drifts by that factor at every rescale.  The empty asm makes the rounded product opaque to the optimiser.
__device__ __forceinline__ float log_scale(const FwdParams& P, float m) {
    float c = P.p * fast_log2(m);
    asm volatile("" : "+v"(c));
    return c;
}

// Sum normalised by a maximum. Everything is kept in the log2 domain: c = p * log2(m), s = sum 2^(p*log2|t| - c).
template <bool GIVEN_MAX>
struct OpNormalized {
    static constexpr int NX = 1, PHASES = GIVEN_MAX ? 1 : 2, NOF = 1, NOI = 0;
    static constexpr bool PREFETCH = false;  // three registers per output: no room for a second operand set
    static constexpr bool PREFETCH_SMALL = true;
    static constexpr bool HEAVY = true;
    static constexpr float COST = GIVEN_MAX ? 25.8f : 35.9f;
    struct Acc { float m, c, s; };
    __device__ static __forceinline__ void init(Acc& a, const FwdParams& P, int kg, int m, int n, int g) {
        if constexpr (GIVEN_MAX) {
            float mx = 1.f;
            if (m < P.s.M && n < P.s.COg) {
                const int b = m / P.s.HW, hw = m - b * P.s.HW;
                mx = P.aux[y_off(P.s, b, g, n, hw)];
            }
            a.m = mx;
            a.c = log_scale(P, mx);
            a.s = kg == 0 ? fast_exp2(log_scale(P, kEps) - a.c) : 0.f;
        } else {
            a.m = kEps;
            a.c = log_scale(P, kEps);
            a.s = kg == 0 ? 1.f : 0.f;  // the phantom term (1e-10 / m)^p with m = 1e-10
        }
    }
    template <int TN>
    __device__ static __forceinline__ void row2(Acc (&a)[TN], const FwdParams& P, int ph, float x0, float,
                                                const float (&w0)[TN], float x1, float, const float (&w1)[TN]) {
        float d0[TN], d1[TN];
#pragma unroll
        for (int j = 0; j < TN; j++) { d0[j] = x0 - w0[j]; d1[j] = x1 - w1[j]; }
        if (!GIVEN_MAX && ph == 0) {
#pragma unroll
            for (int j = 0; j < TN; j++) a[j].m = fmaxf(fmaxf(a[j].m, fabsf(d0[j])), fabsf(d1[j]));
        } else {
#pragma unroll
            for (int j = 0; j < TN; j++) { d0[j] = fast_log2(fabsf(d0[j])); d1[j] = fast_log2(fabsf(d1[j])); }
#pragma unroll
            for (int j = 0; j < TN; j++) { d0[j] = fmaf(P.p, d0[j], -a[j].c); d1[j] = fmaf(P.p, d1[j], -a[j].c); }
#pragma unroll
            for (int j = 0; j < TN; j++) { d0[j] = fast_exp2(d0[j]); d1[j] = fast_exp2(d1[j]); }
#pragma unroll
            for (int j = 0; j < TN; j++) a[j].s += d0[j];
#pragma unroll
            for (int j = 0; j < TN; j++) a[j].s += d1[j];
        }
    }
    __device__ static __forceinline__ void phase_end(Acc& a, const FwdParams& P, int ph, int) {
        if (!GIVEN_MAX && ph == 0) {
            // rescale the sum to the (possibly) new maximum; an unchanged maximum gives the factor 2^0 = 1 exactly
            const float cn = log_scale(P, a.m);
            a.s *= fast_exp2(a.c - cn);
            a.c = cn;
        }
    }
    __device__ static __forceinline__ void merge(Acc& a, const Acc& b, const FwdParams& P) {
        if constexpr (GIVEN_MAX) {
            a.s += b.s;
        } else {
            const float mx = fmaxf(a.m, b.m);
            const float cn = mx == a.m ? a.c : b.c;
            a.s = a.s * fast_exp2(a.c - cn) + b.s * fast_exp2(b.c - cn);
            a.m = mx;
            a.c = cn;
        }
    }
    __device__ static __forceinline__ void finalize(const Acc& a, const FwdParams& P, float* fv, int*) {
        fv[0] = root_p(a.s, P) * a.m;
    }
};

// The normalised sum in one pass, for moderate p: any scale s >= max |x - w| gives the same result,
// out = s * (sum (|t| / s)^p)^(1/p), as long as the sum stays inside the float range.  The scale here depends on the
// row of x only -- its largest magnitude plus the largest magnitude in all of w, prepared as c = p * log2(s) by two
// small kernels -- so it costs one register per row of the micro-tile, no pass for the maxima and no rescaling.
// The scale enters the terms and the result through the same rounded c, so its rounding cancels.  An output whose
// true maximum lies so far below the bound that the sum falls under 2^-90 (its terms near the flush-to-zero range)
// is stored as -1; a pass over the outputs recomputes those with their exact maximum (norm_fixup_kernel).  A NaN
// sum takes the same route.
constexpr float kRowScaledMinSum = 8.0779357e-28f;  // 2^-90
struct OpRowScaled {
    static constexpr int NX = 1, PHASES = 1, NOF = 1, NOI = 0;
    static constexpr bool PREFETCH = true;
    static constexpr float COST = 26.8f;
    struct Acc { float c, s; };  // c is the same for all outputs of a row: the optimiser keeps one copy per row
    __device__ static __forceinline__ void init(Acc& a, const FwdParams& P, int kg, int m, int, int g) {
        const int mm = m < P.s.M ? m : P.s.M - 1;
        a.c = P.aux[(long)mm * P.s.G + g];
        a.s = kg == 0 ? fast_exp2(P.p * fast_log2(kEps) - a.c) : 0.f;  // the reference's floor term (1e-10 / s)^p
    }
    template <int TN>
    __device__ static __forceinline__ void row2(Acc (&a)[TN], const FwdParams& P, int, float x0, float,
                                                const float (&w0)[TN], float x1, float, const float (&w1)[TN]) {
        constexpr int N = 2 * TN;
        float e[N];
#pragma unroll
        for (int j = 0; j < TN; j++) { e[j] = x0 - w0[j]; e[TN + j] = x1 - w1[j]; }
#pragma unroll
        for (int j = 0; j < N; j++) e[j] = fast_log2(fabsf(e[j]));
#pragma unroll
        for (int j = 0; j < N; j++) e[j] = fmaf(P.p, e[j], -a[j % TN].c);
#pragma unroll
        for (int j = 0; j < N; j++) e[j] = fast_exp2(e[j]);
#pragma unroll
        for (int j = 0; j < TN; j++) a[j].s += e[j];
#pragma unroll
        for (int j = 0; j < TN; j++) a[j].s += e[TN + j];
    }
    __device__ static __forceinline__ void phase_end(Acc&, const FwdParams&, int, int) {}
    __device__ static __forceinline__ void merge(Acc& a, const Acc& b, const FwdParams&) { a.s += b.s; }
    __device__ static __forceinline__ void finalize(const Acc& a, const FwdParams& P, float* fv, int*) {
        fv[0] = a.s >= kRowScaledMinSum ? fast_exp2((fast_log2(a.s) + a.c) * P.inv_p) : -1.0f;
    }
};

// The same sum for large p, in one pass and with most pairs skipped.  A pair with |t| < 2^(-32/p) * m adds less than
// 2^-32 to a sum that is at least 1: 5120 dropped pairs change the sum by < 1.2e-6 and the result (its p-th root) by
// that over p.  For large p almost every pair is below that threshold (p = 100: |t| < 0.80 m), so the usual work per
// pair is a subtraction and a compare against t = 2^(-32/p) * (running maximum); log2 / exp2 run only when some lane
// of the wave has a pair above its threshold, and only when some lane exceeds its maximum is the maximum raised and
// the sum rescaled.  The running maximum is never larger than the final one, so nothing is dropped that would have
// counted.  The test is wave-wide for a whole row first (its usual outcome, "nothing counts", must be the
// fall-through: taken branches are expensive), then per output column.
template <bool GIVEN_MAX>
struct OpNormSkip {
    static constexpr int NX = 1, PHASES = 1, NOF = 1, NOI = 0;
    static constexpr bool PREFETCH = false;
    static constexpr bool TILE_BOUND = true;
    static constexpr float COST = 10.f;
    // c = p * log2(running maximum), s = the sum relative to it, t = threshold = thr * maximum.  The maximum itself
    // is not kept (three registers per output leave the 1024-thread tile without spills): where it is needed it is
    // t / thr, and the lanes whose maximum stays keep c bit for bit (see raise_max).
    struct Acc { float c, s, t; };
    __device__ static __forceinline__ void init(Acc& a, const FwdParams& P, int kg, int m, int n, int g) {
        typename OpNormalized<GIVEN_MAX>::Acc b;
        OpNormalized<GIVEN_MAX>::init(b, P, kg, m, n, g);
        if constexpr (!GIVEN_MAX) {
            // Seed of the running maximum: the larger of the pairs at the k where this row of x, and where this row
            // of w, is largest.  Any pair of the reduction is a valid starting point (the maximum is only a scale,
            // and it is still raised whenever a pair exceeds it); these are close to the final maximum, so the
            // thresholds are tight from the first k on instead of after a long warm-up in which almost every pair
            // "counts".  A small kernel of its own computes the seeds (norm_seed_outputs_kernel).
            if (P.aux != nullptr && m < P.s.M && n < P.s.COg) {
                const int bb = m / P.s.HW, hw = m - bb * P.s.HW;
                b.m = P.aux[y_off(P.s, bb, g, n, hw)];
                b.c = log_scale(P, b.m);
                b.s = kg == 0 ? fast_exp2(log_scale(P, kEps) - b.c) : 0.f;
            }
        }
        a.c = b.c;
        a.s = b.s;
        a.t = b.m * P.thr;
        // outputs of the tile's padding (never stored): no pair counts, so that they cannot send their wave into the
        // slow path at every step
        if (!(m < P.s.M && n < P.s.COg)) a.t = __builtin_inff();
    }
    template <int TN>
    __device__ static __forceinline__ void row2(Acc (&a)[TN], const FwdParams& P, int, float x0, float,
                                                const float (&w0)[TN], float x1, float, const float (&w1)[TN]) {
        unsigned long long hot[TN], any = 0;  // wave-wide masks: straight from the compares, no vector round trip
#pragma unroll
        for (int j = 0; j < TN; j++) {
            const float e = fmaxf(fabsf(x0 - w0[j]), fabsf(x1 - w1[j]));
            hot[j] = __builtin_amdgcn_ballot_w64(e > a[j].t);
            any |= hot[j];
        }
        if (__builtin_expect(any != 0, 0)) {
            // (the differences are formed again here, from copies the compiler cannot identify with x0 and x1:
            // kept from above they would occupy 3 * TN registers across the branch and push accumulators into scratch)
            float xa = x0, xb = x1;
            asm volatile("" : "+v"(xa), "+v"(xb));
#pragma unroll
            for (int j = 0; j < TN; j++) {
                if (hot[j] != 0) {  // some lane has a pair that counts
                    const float d0 = xa - w0[j], d1 = xb - w1[j];
                    if constexpr (!GIVEN_MAX) {
                        const float e = fmaxf(fabsf(d0), fabsf(d1));
                        const float et = e * P.thr;  // above the maximum <=> et above the threshold
                        if (__builtin_amdgcn_ballot_w64(et > a[j].t) != 0) raise_max(a[j], P, e, et);
                    }
                    const float e0 = fast_exp2(fmaf(P.p, fast_log2(fabsf(d0)), -a[j].c));
                    const float e1 = fast_exp2(fmaf(P.p, fast_log2(fabsf(d1)), -a[j].c));
                    a[j].s += e0;
                    a[j].s += e1;
                }
            }
        }
    }
    // Whole k-tile at once: bx / bw are the largest |x| of my rows and the largest |w| of my columns inside the tile
    // (infinite when the launcher supplied no bounds: nothing is skipped then).  |x - w| <= bx + bw, so when that
    // stays at or below the threshold of every output of the wave no pair of the tile counts, and none raises a
    // maximum either (the thresholds are below the maxima).
    template <int TM, int TN>
    __device__ static __forceinline__ bool tile_skip(const Acc (&a)[TM][TN], const float (&bx)[TM], const float (&bw)[TN]) {
        bool hot = false;
#pragma unroll
        for (int i = 0; i < TM; i++)
#pragma unroll
            for (int j = 0; j < TN; j++) hot |= bx[i] + bw[j] > a[i][j].t;
        return __builtin_amdgcn_ballot_w64(hot) == 0;
    }
    // some lane of the wave exceeds its maximum (et = e * thr above its threshold): raise it and rescale the sum;
    // the lanes whose maximum stays keep c bit for bit, so their factor is 2^0 = 1 exactly
    __device__ static __forceinline__ void raise_max(Acc& a, const FwdParams& P, float e, float et) {
        const bool up = et > a.t;
        const float cn = up ? log_scale(P, e) : a.c;
        a.s *= fast_exp2(a.c - cn);
        a.c = cn;
        a.t = up ? et : a.t;
    }
    __device__ static __forceinline__ void phase_end(Acc&, const FwdParams&, int, int) {}
    __device__ static __forceinline__ void merge(Acc& a, const Acc& b, const FwdParams&) {
        if constexpr (GIVEN_MAX) {
            a.s += b.s;
        } else {
            const float cn = fmaxf(a.c, b.c);
            a.s = a.s * fast_exp2(a.c - cn) + b.s * fast_exp2(b.c - cn);
            a.c = cn;
            a.t = fmaxf(a.t, b.t);
        }
    }
    __device__ static __forceinline__ void finalize(const Acc& a, const FwdParams& P, float* fv, int*) {
        fv[0] = root_p(a.s, P) * (a.t * P.inv_thr);
    }
};

}  // namespace ndist
