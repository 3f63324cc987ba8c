// Backward of the finite-p distance, both gradients in one pass over the (row, co, ci) iteration space.
// Replaces norm_dist<ip>::backward_input and ::backward_input_weight of the reference
// (core/cuda/norm_dist_cuda.cu:238-509,566-623; exponent p-1 from core/cuda/norm_dist.cpp:66-91):
//
//   term(m, co, ci) = g[m, co] * sign(t) * (|t| / out[m, co])^(p-1),  t = x[m, ci] - w[co, ci],  m = (b, hw)
//   grad_x[m, ci]  =  sum_co term          grad_w[co, ci] = -sum_m term
//
// Neither gradient reduces over ci, so ci is spread over the 64 lanes of a wave and BOTH reductions run serially
// inside a lane: a lane keeps x[m, ci] and the grad_x accumulators of BT rows in registers, walks over co, loads
// w[co, ci] once per co (one coalesced row segment per wave), and accumulates its grad_w partial for that co over
// its BT rows.  The per-(m, co) factors 1/out and g do not depend on ci, i.e. they are uniform over the wave: a
// small pre-pass writes them transposed ([co][m], so consecutive rows are consecutive in memory) and the main
// loop fetches them with scalar loads into SGPRs.  No cross-lane traffic and no LDS operand traffic at all; per
// (m, co, ci): one subtract, one scale, the power ladder, and two fused multiply-adds.
//
// A workgroup is NW waves working on NW*BT consecutive rows and the same 64-wide ci slab; their grad_w partials
// meet in LDS (one slot per wave, summed after a barrier) and are written once per (16 co x 64 ci) unit.  Workgroups are persistent and take an
// equal, contiguous share of the units (order: group, slab, row chunk, co chunk), so that grad_x accumulators stay
// in registers while consecutive units share their rows; they are added to global memory when the rows change.
#pragma once
#include <type_traits>

#include "ndist_common.h"

namespace ndist {

constexpr int kBwdCoUnit = 16;  // co per unit
constexpr int kBwdSlab = 64;    // ci per unit == lanes of a wave

// Pointer arguments of the main kernel are passed individually and __restrict__-qualified: the compiler must know
// that the stores to the gradients cannot alias the factor array, or it will not fetch it through the scalar cache.
//   aT [G*COg][Mpad]  the per-(row, co) factor, transposed so that consecutive rows are consecutive in memory:
//                       p = 1      grad_output                      (term = a * sign(t))
//                       p > 1      sign(g) * |g|^(1/(p-1)) / out     (term = sign(v) * |v|^(p-1), v = a * t)
//                     folding grad_output into the factor as its (p-1)-th root leaves ONE wave-uniform operand per
//                     term; v stays in range because |t / out| <= 1 and the root compresses |g| towards 1
//   gx  accumulated with atomics: zeroed by the caller
//   gw  written (one row chunk) or accumulated with atomics (several: zeroed by the caller)
struct BwdParams {
    Geom s;
    int Mpad;         // rows padded to a multiple of NW*BT; padding carries g = 0
    int nslab, ncc, nrc;
    int gw_add;       // grad_weight is added to (atomics into a gradient zeroed beforehand): several row chunks, or a
                      // caller that accumulates over several launches; 0: stored
    long total;       // G * nslab * nrc * ncc units
    float q;          // p - 1
    // term-skipping variant (IP == -3): terms below 2^-40 * max|grad_output| are dropped; gmax points at that maximum
    // (written by the pre-pass).  Optional gate as in the forward: run only when (gate[0] < gate_limit) == gate_sense.
    const float* gmax;
    const int* gate;
    int gate_limit, gate_sense;
    // second gate of the same form: chooses between the two skipping variants (term by term, or by bounds first)
    const int* gate2;
    int gate2_limit, gate2_sense;
    long g_off;       // offset in floats from the factors to a second array of the same layout, 0 if there is none:
                      // grad_output (IP -2, whose factors are 1/out), or the part of every factor that float32
                      // dropped (IP -5, and the rare branch of the skipping variants -3 / -4)
    // Reproducible grad_input (row-split kernel): a workgroup that holds ALL units of a (group, slab, row chunk) block
    // stores that block's grad_input directly; a block shared between neighbouring workgroups goes into `part`
    // ([workgroup][2][rows per workgroup][64]: slot 0 for the block a workgroup starts in, slot 1 for the one it ends
    // in) and bwd_gx_fixup_kernel adds the shares in workgroup order.  nullptr: global atomic adds into a zeroed
    // grad_input (sums in arrival order).
    float* part;
    // Rows that are the patches of images (convolutional layer): when `image` is set, row m = (sample, output position)
    // is not read from memory laid out [M][CI] but gathered from the images [B][C][H][W] of geometry `cv`, zeros
    // outside the image, column ci of group g being tap (g * CIg + ci) of the unfolded problem.  Main kernel only.
    // The description lives in device memory, not among the kernel's arguments: its fields are then fetched where the
    // rows change and nowhere else (as arguments they cost the main loop scalar registers it does not have).
    const struct BwdImage* image;
};
struct BwdImage {
    const float* img;
    UnfoldGeom cv;
};
static_assert(sizeof(BwdImage) == 64 && offsetof(BwdImage, cv) == 8, "read below as sixteen words");

typedef float f16v __attribute__((ext_vector_type(16)));
// 16 consecutive factors through the scalar data cache: a load from the constant address space with a wave-uniform
// address is always selected as s_load_dwordx16.  The factor array is written by an earlier kernel and only read
// here, which is what the constant address space promises.
__device__ __forceinline__ f16v load_factors(const float* p) {
    typedef const f16v __attribute__((address_space(4))) * cptr;
    return *reinterpret_cast<cptr>(reinterpret_cast<uintptr_t>(p));
}
typedef float f8v __attribute__((ext_vector_type(8)));
__device__ __forceinline__ f8v load_factors8(const float* p) {
    typedef const f8v __attribute__((address_space(4))) * cptr;
    return *reinterpret_cast<cptr>(reinterpret_cast<uintptr_t>(p));
}
constexpr int kBwdRowBatch = 16;  // rows whose factors are fetched by one 16-dword scalar load


// one (row, co, ci) term for a row slot of the lane, given the wave-uniform factor of that (row, co)
// R terms (R consecutive row slots of the lane, one co) given the wave-uniform factors of those (row, co) pairs.
// IP: 0..8 the exponent p-1 by repeated multiplication; -1 / -3 general exponent >= 1 (grad_output folded into the
// factor); -2 general exponent < 1, where the root that folds grad_output could overflow: `a` is 1/out and
// grad_output comes separately in `g2`; -5 general exponent >= 1 with a compensated product (large exponents): `g2`
// is the part of the factor that float32 dropped.
// Large exponents multiply every rounding under the power by q = p - 1: with v = fl(t * a) and a = fl(a_exact) the
// term carries q * (two roundings) on top of the rounding of t = x - w that no float32 evaluation avoids, which at
// q = 200 is 1 - 2e-5 relative against the 1e-5 the operator is held to.  Both are known exactly:
// e = fma(t, a, -v) + t * a_lo is what v is missing (a_lo from the pre-pass, which forms the factor in double
// precision), and sign(v + e)|v + e|^q = |v|^(q-1) * (v + q e) to first order: three more instructions (+ 29 % on
// the kernel), used by the plain variant from q = 64 on (-5).  The skipping variants (-3, -4) evaluate their few
// surviving terms uncompensated: with the correction inlined into their unrolled bodies the register allocation of
// the bounds variant went from 48 to 600 - 1000 spilled registers (also with the correction behind a second,
// rarer test, and as a real call), and both variants lost 35 - 100 % of their speed.
// The arithmetic is laid out in stages over the R rows: back-to-back dependent vector instructions stall a wave,
// independent neighbours do not.
template <int IP, bool WITH_W, int R>
__device__ __forceinline__ void bwd_terms(const float* __restrict__ xv, float wv, const float (&a)[R], const float (&g2)[R],
                                          float q, float thr, float* __restrict__ gxa, float (&gwp)[R]) {
    float t[R];
#pragma unroll
    for (int r = 0; r < R; r++) t[r] = xv[r] - wv;
    if constexpr (IP == -2) {
        float e[R];
#pragma unroll
        for (int r = 0; r < R; r++) e[r] = fast_log2(fabsf(t[r]) * a[r]);
#pragma unroll
        for (int r = 0; r < R; r++) e[r] = fast_exp2(q * e[r]);
#pragma unroll
        for (int r = 0; r < R; r++) e[r] = __builtin_copysignf(e[r], t[r]);
#pragma unroll
        for (int r = 0; r < R; r++) gxa[r] = fmaf(g2[r], e[r], gxa[r]);
        if (WITH_W) {
#pragma unroll
            for (int r = 0; r < R; r++) gwp[r] = fmaf(g2[r], e[r], gwp[r]);
        }
    } else if constexpr (IP == 0) {
        // p = 1: g * sign(t), sign(0) = +1
#pragma unroll
        for (int r = 0; r < R; r++) t[r] = t[r] >= 0.f ? a[r] : -a[r];
#pragma unroll
        for (int r = 0; r < R; r++) gxa[r] += t[r];
        if (WITH_W) {
#pragma unroll
            for (int r = 0; r < R; r++) gwp[r] += t[r];
        }
    } else if constexpr (IP == -3) {
        // general exponent with skipping (large q): |v|^q < 2^-40 * max|g| cannot be seen in a gradient whose large
        // elements are of the order of max|g|, and for large q that holds for almost every term.  The usual work per
        // term is sub, scale, compare; the wave-wide test is made for the whole group first (its usual outcome,
        // "nothing counts", is the fall-through), then per row.
        const float q1 = q - 1.0f;
        unsigned long long hot[R], any = 0;
#pragma unroll
        for (int r = 0; r < R; r++) t[r] = t[r] * a[r];
#pragma unroll
        for (int r = 0; r < R; r++) {
            hot[r] = __builtin_amdgcn_ballot_w64(fabsf(t[r]) > thr);
            any |= hot[r];
        }
        if (__builtin_expect(any != 0, 0)) {
#pragma unroll
            for (int r = 0; r < R; r++) {
                if (hot[r] != 0) {
                    const float e = fast_exp2(q1 * fast_log2(fabsf(t[r])));
                    gxa[r] = fmaf(t[r], e, gxa[r]);
                    if (WITH_W) gwp[r] = fmaf(t[r], e, gwp[r]);
                }
            }
        }
    } else if constexpr (IP == -5) {
        // IP -1 with the compensated product: g2 = a_lo
        float e[R], v[R], miss[R];
        const float q1 = q - 1.0f;
#pragma unroll
        for (int r = 0; r < R; r++) v[r] = t[r] * a[r];
#pragma unroll
        for (int r = 0; r < R; r++) miss[r] = fmaf(t[r], a[r], -v[r]);
#pragma unroll
        for (int r = 0; r < R; r++) e[r] = fast_log2(fabsf(v[r]));
#pragma unroll
        for (int r = 0; r < R; r++) miss[r] = fmaf(t[r], g2[r], miss[r]);
#pragma unroll
        for (int r = 0; r < R; r++) e[r] = fast_exp2(q1 * e[r]);
#pragma unroll
        for (int r = 0; r < R; r++) v[r] = fmaf(q, miss[r], v[r]);
#pragma unroll
        for (int r = 0; r < R; r++) gxa[r] = fmaf(v[r], e[r], gxa[r]);
        if (WITH_W) {
#pragma unroll
            for (int r = 0; r < R; r++) gwp[r] = fmaf(v[r], e[r], gwp[r]);
        }
    } else if constexpr (IP == -1) {
        // general exponent q >= 1: sign(v)|v|^q = v * |v|^(q-1), the power through the hardware exp2 / log2 and the
        // sign for free from the last multiplication, which is fused into the two accumulations.  The factor already
        // carries |g|^(1/q) and the normalisation by out, so the dominant terms have a logarithm near log2|g|/q and
        // stay accurate for large q.  v = 0: log2 gives -inf, exp2 gives 0 (q > 1 on this path).
        float e[R];
        const float q1 = q - 1.0f;
#pragma unroll
        for (int r = 0; r < R; r++) t[r] = t[r] * a[r];
#pragma unroll
        for (int r = 0; r < R; r++) e[r] = fast_log2(fabsf(t[r]));
#pragma unroll
        for (int r = 0; r < R; r++) e[r] = fast_exp2(q1 * e[r]);
#pragma unroll
        for (int r = 0; r < R; r++) gxa[r] = fmaf(t[r], e[r], gxa[r]);
        if (WITH_W) {
#pragma unroll
            for (int r = 0; r < R; r++) gwp[r] = fmaf(t[r], e[r], gwp[r]);
        }
    } else if constexpr (IP == 1) {
#pragma unroll
        for (int r = 0; r < R; r++) t[r] = t[r] * a[r];
#pragma unroll
        for (int r = 0; r < R; r++) gxa[r] += t[r];
        if (WITH_W) {
#pragma unroll
            for (int r = 0; r < R; r++) gwp[r] += t[r];
        }
    } else {
        // v = a * t ; sign(v)|v|^IP = lo * hi, the last multiplication fused into the two accumulations
        float lo[R], hi[R];
#pragma unroll
        for (int r = 0; r < R; r++) lo[r] = t[r] * a[r];
        if constexpr (IP == 2) {
#pragma unroll
            for (int r = 0; r < R; r++) hi[r] = fabsf(lo[r]);
        } else if constexpr (IP == 3) {
#pragma unroll
            for (int r = 0; r < R; r++) hi[r] = lo[r] * lo[r];
        } else if constexpr (IP == 4) {
#pragma unroll
            for (int r = 0; r < R; r++) hi[r] = lo[r] * lo[r];
#pragma unroll
            for (int r = 0; r < R; r++) lo[r] = lo[r] * fabsf(lo[r]);
        } else if constexpr (IP == 5) {
#pragma unroll
            for (int r = 0; r < R; r++) hi[r] = lo[r] * lo[r];
#pragma unroll
            for (int r = 0; r < R; r++) hi[r] = hi[r] * hi[r];
        } else if constexpr (IP == 6) {
            float v2[R];
#pragma unroll
            for (int r = 0; r < R; r++) v2[r] = lo[r] * lo[r];
#pragma unroll
            for (int r = 0; r < R; r++) { hi[r] = v2[r] * v2[r]; lo[r] = lo[r] * fabsf(lo[r]); }
        } else if constexpr (IP == 8) {
            // sign(v)|v|^8 = (v |v|) * v^6
            float v2[R];
#pragma unroll
            for (int r = 0; r < R; r++) v2[r] = lo[r] * lo[r];
#pragma unroll
            for (int r = 0; r < R; r++) hi[r] = v2[r] * v2[r];
#pragma unroll
            for (int r = 0; r < R; r++) { hi[r] = hi[r] * v2[r]; lo[r] = lo[r] * fabsf(lo[r]); }
        } else {
            float v2[R];
#pragma unroll
            for (int r = 0; r < R; r++) v2[r] = lo[r] * lo[r];
#pragma unroll
            for (int r = 0; r < R; r++) v2[r] = v2[r] * lo[r];
#pragma unroll
            for (int r = 0; r < R; r++) hi[r] = v2[r] * v2[r];
        }
#pragma unroll
        for (int r = 0; r < R; r++) gxa[r] = fmaf(lo[r], hi[r], gxa[r]);
        if (WITH_W) {
#pragma unroll
            for (int r = 0; r < R; r++) gwp[r] = fmaf(lo[r], hi[r], gwp[r]);
        }
    }
}

// decoded position of a unit: group, ci slab, row chunk, co range
struct BwdUnit {
    long sr;  // index of the (group, slab, row chunk) triple: x rows and grad_x accumulators live as long as it
    int g, ci0, rc, co0, co1;
};
__device__ __forceinline__ BwdUnit bwd_decode(const BwdParams& P, long u) {
    BwdUnit d;
    const int cc = (int)(u % P.ncc);
    d.sr = u / P.ncc;
    d.rc = (int)(d.sr % P.nrc);
    const int gs = (int)(d.sr / P.nrc);
    d.g = gs / P.nslab;
    d.ci0 = (gs - d.g * P.nslab) * kBwdSlab;
    d.co0 = cc * kBwdCoUnit;
    d.co1 = min(d.co0 + kBwdCoUnit, P.s.COg);
    return d;
}

template <int IP, bool WITH_W, int BT, int NW>
__global__ __launch_bounds__(64 * NW, 4) void bwd_fused_kernel(const float* __restrict__ X, const float* __restrict__ W,
                                                            const float* __restrict__ AT, float* __restrict__ GX,
                                                            float* __restrict__ GW, const BwdParams P) {
    constexpr int NT = 64 * NW;
    constexpr int RB = kBwdRowBatch, NB = BT / RB;
    static_assert(BT % RB == 0, "rows per wave must be whole scalar batches");
    // grad_weight partials of the waves meet in LDS.  LDS float atomic adds are far too slow on this hardware
    // (about 190 cycles per wave instruction against 4 for a store), so every wave stores its partial into a slot of
    // its own and, after the barrier that ends the unit, each thread sums the NW slots of its cells.  Two buffers:
    // a buffer is rewritten only after the next unit's barrier, when all of its readers are done.
    constexpr int SLOT = kBwdCoUnit * kBwdSlab;  // floats per wave per buffer == weights of a unit
    // IP == -4, where most (wave, co) pairs have nothing to add: a wave stores only the partials that exist and sets
    // its bit in the co's word of `hotmask` (integer LDS atomics are fast); the reducer reads the slots named there.
    __shared__ float slots[WITH_W ? 2 * NW * SLOT : 1];
    __shared__ unsigned hotmask[(WITH_W && IP == -4) ? 2 * kBwdCoUnit : 1];
    static_assert(IP != -4 || NW <= 32, "one bit per wave");
    const Geom& s = P.s;
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);

    if (P.gate != nullptr && ((P.gate[0] < P.gate_limit) != (P.gate_sense != 0))) return;
    if (P.gate2 != nullptr && ((P.gate2[0] < P.gate2_limit) != (P.gate2_sense != 0))) return;
    // drop threshold on |v| of the skipping variant: |v|^q < 2^-40 * max|g|
    const float thr = (IP == -3 || IP == -4) ? fast_exp2((fast_log2(P.gmax[0]) - 40.0f) / P.q) : 0.f;

    const long u_begin = (long)blockIdx.x * P.total / gridDim.x;
    const long u_end = (long)(blockIdx.x + 1) * P.total / gridDim.x;
    if (u_begin >= u_end) return;

    float xv[BT], gxa[BT];
    // IP == -4 (skipping by bounds): lane r < BT holds the largest |x| of row r over the slab; the largest |w| of
    // every co of a unit over the slab comes through LDS from the wave that staged that co
    float xmaxv = 0.f;
    __shared__ float wmaxbuf[2 * kBwdCoUnit];
    BwdUnit cur = bwd_decode(P, u_begin);
    long loaded_sr = -1;
    int xg = 0, xci = 0, xr0 = 0;  // group, ci and first row of the rows held in xv / gxa
    bool x_ok = false;

    auto flush_gx = [&]() {
        if (!x_ok) return;
        // (the skipping variants are only ever queued next to other variants, where `part` is not used: they keep
        // the plain atomic path, and their register budget)
        constexpr bool kShares = IP != -3 && IP != -4;
        bool sole = false;
        if constexpr (kShares) {
            const long b0 = loaded_sr * P.ncc;
            sole = P.part != nullptr && u_begin <= b0 && b0 + P.ncc <= u_end;  // all units of the block are mine
            if (P.part != nullptr && !sole) {
                const int slot = loaded_sr == u_begin / P.ncc ? 0 : 1;
                float* __restrict__ dst = P.part + (((long)blockIdx.x * 2 + slot) * (NW * BT) + wave * BT) * kBwdSlab + lane;
#pragma unroll
                for (int i = 0; i < BT; i++) dst[i * kBwdSlab] = gxa[i];
                return;
            }
        }
#pragma unroll
        for (int i = 0; i < BT; i++) {
            const int m = xr0 + i;
            if (m < s.M) {
                const int b = m / s.HW, hw = m - b * s.HW;
                float* __restrict__ dst = GX + x_off(s, b, xg, xci, hw);
                if (sole) *dst = gxa[i];
                else atomicAdd(dst, gxa[i]);
            }
        }
    };
    auto factor_ptr = [&](const BwdUnit& d) -> const float* {
        return AT + ((long)(d.g * s.COg + d.co0) * P.Mpad + (long)(d.rc * NW + wave) * BT);
    };
    // The 16 co x 64 ci weights of a unit are the same for every wave of the workgroup: they are fetched once per
    // unit (one or two elements per thread, a unit ahead), parked in registers during the unit, stored to LDS
    // before the barrier that ends it, and read from there one co ahead.  Indices beyond the slab or the co range
    // are clamped (their results are never stored), so every load is unconditional.
    constexpr int WPT = SLOT / NT;
    static_assert(SLOT % NT == 0, "unit weights must divide over the threads");
    __shared__ float wbuf[2 * SLOT];
    auto fetch_w = [&](const BwdUnit& d, float (&r)[WPT]) {
#pragma unroll
        for (int j = 0; j < WPT; j++) {
            const int e = threadIdx.x + j * NT;
            const int co = min(d.co0 + (e >> 6), d.co1 - 1), ci = min(d.ci0 + (e & 63), s.CIg - 1);
            r[j] = W[w_off(s, d.g, co, ci)];
        }
    };
    auto store_w = [&](int buf, const float (&r)[WPT]) {
#pragma unroll
        for (int j = 0; j < WPT; j++) wbuf[buf * SLOT + threadIdx.x + j * NT] = r[j];
        if constexpr (IP == -4) {
            // element threadIdx.x + j * NT lies in co row wave + j * NW of the unit: a wave stages whole rows
            static_assert(IP != -4 || WPT * NW == kBwdCoUnit, "the waves stage the co rows of the unit");
#pragma unroll
            for (int j = 0; j < WPT; j++) {
                float m = fabsf(r[j]);
#pragma unroll
                for (int d = 32; d >= 1; d >>= 1) m = fmaxf(m, __shfl_xor(m, d, 64));
                if (lane == 0) wmaxbuf[buf * kBwdCoUnit + wave + j * NW] = m;
            }
        }
    };
    // factors (first row batch) and weight of the first co of the first unit; afterwards they are always requested
    // one batch / one co ahead, across unit boundaries too
    const float* __restrict__ ap = factor_ptr(cur);
    f16v a_cur = load_factors(ap);
    f16v g_cur = a_cur;
    if constexpr (IP == -2 || IP == -5) g_cur = load_factors(ap + P.g_off);
    {
        float w0[WPT];
        fetch_w(cur, w0);
        store_w((int)(u_begin & 1), w0);
        if constexpr (IP == -4 && WITH_W) {
            if (threadIdx.x < 2 * kBwdCoUnit) hotmask[threadIdx.x] = 0u;
        }
        __syncthreads();
    }

    // IP == -4: factor vectors of four co in flight (lane r < BT: factor of row r), see the co loop
    float avq[4] = {0.f, 0.f, 0.f, 0.f};
    // lanes 0..31: factors of co 2 * pair, lanes 32..63: of co 2 * pair + 1 (rows lane & 31)
    const int half = lane >> 5;
    auto load_av = [&](const float* __restrict__ base, int pair, int nco) __attribute__((always_inline)) -> float {
        const int cl = 2 * pair + half;
        return ((lane & 31) < BT && cl < nco) ? base[(long)cl * P.Mpad + (lane & 31)] : 0.f;
    };
    if constexpr (IP == -4) {
#pragma unroll
        for (int k = 0; k < 4; k++) avq[k] = load_av(factor_ptr(cur), k, cur.co1 - cur.co0);
    }

    for (long u = u_begin; u < u_end; u++) {
        const bool has_next = u + 1 < u_end;
        const BwdUnit nxt = bwd_decode(P, has_next ? u + 1 : u);
        float wstage[WPT];
        fetch_w(nxt, wstage);  // consumed at the end of this unit
        const float* __restrict__ wl = wbuf + (int)(u & 1) * SLOT + lane;
        float wnext = wl[0];
        if (cur.sr != loaded_sr) {
            if (loaded_sr >= 0) flush_gx();
            loaded_sr = cur.sr;
            xg = cur.g;
            xci = cur.ci0 + lane;
            x_ok = xci < s.CIg;
            xr0 = (cur.rc * NW + wave) * BT;
            if (P.image != nullptr) {
                typedef int i16v __attribute__((ext_vector_type(16)));
                typedef const i16v __attribute__((address_space(4))) * cptr;
                const i16v raw = *reinterpret_cast<cptr>(reinterpret_cast<uintptr_t>(P.image));  // one scalar load
                const float* __restrict__ img = reinterpret_cast<const float*>(
                    ((unsigned long long)(unsigned)raw[1] << 32) | (unsigned long long)(unsigned)raw[0]);
                UnfoldGeom cv;
                cv.B = raw[2], cv.C = raw[3], cv.H = raw[4], cv.W = raw[5], cv.kh = raw[6], cv.kw = raw[7];
                cv.dh = raw[8], cv.dw = raw[9], cv.ph = raw[10], cv.pw = raw[11], cv.sh = raw[12], cv.sw = raw[13];
                cv.OH = raw[14], cv.OW = raw[15];
                // the lane's tap: channel and pixel offset inside the window (once per change of rows)
                const int col = xg * s.CIg + xci, taps = cv.kh * cv.kw;
                const int c = col / taps, tap = col - c * taps;
                const int ti = tap / cv.kw, tj = tap - ti * cv.kw;
                const int hi = ti * cv.dh - cv.ph, wj = tj * cv.dw - cv.pw;
                const long lane_off = ((long)c * cv.H + hi) * cv.W + wj;
                // the wave's first row: sample and output position, stepped from row to row
                const int L = cv.OH * cv.OW;
                int b = xr0 / L, oh = (xr0 - b * L) / cv.OW, ow = xr0 - b * L - oh * cv.OW;
#pragma unroll
                for (int i = 0; i < BT; i++) {
                    gxa[i] = 0.f;
                    xv[i] = 0.f;
                    const int h0 = oh * cv.sh, w0 = ow * cv.sw;
                    if (x_ok && xr0 + i < s.M && (unsigned)(h0 + hi) < (unsigned)cv.H && (unsigned)(w0 + wj) < (unsigned)cv.W)
                        xv[i] = img[((long)b * cv.C * cv.H + h0) * cv.W + w0 + lane_off];
                    if (++ow == cv.OW) {
                        ow = 0;
                        if (++oh == cv.OH) {
                            oh = 0;
                            b++;
                        }
                    }
                }
            } else {
#pragma unroll
                for (int i = 0; i < BT; i++) {
                    const int m = xr0 + i;
                    gxa[i] = 0.f;
                    xv[i] = 0.f;
                    if (x_ok && m < s.M) {
                        const int b = m / s.HW, hw = m - b * s.HW;
                        xv[i] = X[x_off(s, b, xg, xci, hw)];
                    }
                }
            }
            if constexpr (IP == -4) {
#pragma unroll
                for (int i = 0; i < BT; i++) {
                    float m = fabsf(xv[i]);
#pragma unroll
                    for (int d = 32; d >= 1; d >>= 1) m = fmaxf(m, __shfl_xor(m, d, 64));
                    xmaxv = (lane & 31) == i ? m : xmaxv;  // both halves of the wave: two co are tested at once
                }
            }
        }
        float* __restrict__ mine = slots + (WITH_W ? ((int)(u & 1) * NW + wave) * SLOT : 0) + lane;
        const float* __restrict__ ap_next_unit = factor_ptr(nxt);
        if constexpr (IP == -4) {
            // Skipping by bounds.  |v| = |a| |x - w| <= |a| (max|x| + max|w|) over the slab: one vector instruction
            // tests all BT rows of a co (lane r holds the factor and the bound of row r), and only the groups of four
            // rows that may hold a term above the threshold are looked at term by term (the same code as IP == -3,
            // their factors moved to scalar registers with v_readlane).
            static_assert(IP != -4 || BT <= 32, "one mask bit per row");
            const float* __restrict__ arow = factor_ptr(cur);
            const int nco = cur.co1 - cur.co0;
            const float* __restrict__ wmx = wmaxbuf + (int)(u & 1) * kBwdCoUnit + half;
            unsigned stored = 0;  // wave-uniform: the co of this unit for which the wave has stored a partial sum
            // one co of a pair: the groups of four rows whose bit is set, term by term
            auto co_hot = [&](int cl, float av, unsigned mask, int lane0) __attribute__((always_inline)) {
                const float wv = wl[cl * kBwdSlab];
                float gwp[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int q0 = 0; q0 < BT; q0 += 4) {
                    if ((mask >> q0) & 0xFu) {
                        float ga[4];
#pragma unroll
                        for (int r = 0; r < 4; r++)
                            ga[r] = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(av), lane0 + q0 + r));
                        bwd_terms<-3, WITH_W, 4>(&xv[q0], wv, ga, ga, P.q, thr, &gxa[q0], gwp);
                    }
                }
                if (WITH_W) {
                    mine[cl * kBwdSlab] = (gwp[0] + gwp[1]) + (gwp[2] + gwp[3]);
                    stored |= 1u << cl;
                }
            };
            auto pair_body = [&](int pair, float av) __attribute__((always_inline)) {
                const int cl = 2 * pair;
                const float wm = wmx[min(cl, kBwdCoUnit - 2)];  // lanes 32..63 read the entry of co + 1
                const unsigned long long mask = __builtin_amdgcn_ballot_w64(fabsf(av) * (xmaxv + wm) > thr);
                if (__builtin_expect(mask != 0, 0)) {
                    if ((unsigned)mask != 0) co_hot(cl, av, (unsigned)mask, 0);
                    if ((unsigned)(mask >> 32) != 0) co_hot(cl + 1, av, (unsigned)(mask >> 32), 32);
                }
            };
            // the factor vectors are requested four pairs ahead (a rotating set of four registers)
            const int npair = (nco + 1) / 2;
            for (int c4 = 0; c4 < npair; c4 += 4) {
#pragma unroll
                for (int k = 0; k < 4; k++) {
                    const int pair = c4 + k;
                    if (pair < npair) {
                        const float av = avq[k];
                        avq[k] = load_av(arow, pair + 4, nco);
                        pair_body(pair, av);
                    }
                }
            }
            if (WITH_W && stored != 0) {
                if (lane < kBwdCoUnit && ((stored >> lane) & 1u))
                    atomicOr(&hotmask[(int)(u & 1) * kBwdCoUnit + lane], 1u << wave);
            }
            // the first four of the next unit: in flight during the barrier and the grad_weight reduction below
            {
                const int nn = nxt.co1 - nxt.co0;
#pragma unroll
                for (int k = 0; k < 4; k++) avq[k] = load_av(ap_next_unit, k, nn);
            }
        } else if (xr0 >= s.M) {
            // every row of this wave is padding of the last row chunk (x and the factors are zero there): nothing to
            // add; its grad_weight slots read as zero, and the factor requests go on with the next unit's first batch
            if (WITH_W) {
                for (int c = 0; c < cur.co1 - cur.co0; c++) mine[c * kBwdSlab] = 0.f;
            }
            ap = ap_next_unit;
            a_cur = load_factors(ap);
            g_cur = a_cur;
            if constexpr (IP == -2 || IP == -5) g_cur = load_factors(ap + P.g_off);
        } else
        for (int co = cur.co0; co < cur.co1; co++) {
            const float wv = wnext;
            const bool last_co = co + 1 == cur.co1;
            // weight of the next co, from LDS (after the last co: a harmless re-read)
            wnext = wl[min(co + 1 - cur.co0, kBwdCoUnit - 1) * kBwdSlab];
            // one grad_weight partial per row of a stage group: four independent accumulation chains
            float gwp[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int bi = 0; bi < NB; bi++) {
                constexpr int RG = 4;  // rows per stage group
                float fa[RB], fg[RB];
#pragma unroll
                for (int r = 0; r < RB; r++) { fa[r] = a_cur[r]; fg[r] = g_cur[r]; }
                auto group = [&](int q0) {
                    float ga[RG], gg[RG];
#pragma unroll
                    for (int r = 0; r < RG; r++) { ga[r] = fa[q0 + r]; gg[r] = fg[q0 + r]; }
                    bwd_terms<IP, WITH_W, RG>(&xv[bi * RB + q0], wv, ga, gg, P.q, thr, &gxa[bi * RB + q0], gwp);
                };
                // first rows of the batch: their use of the factors is where the wait for the pending request lands
                group(0);
                __builtin_amdgcn_sched_barrier(0);
                // request the next batch now (same co, next rows; or the next co, which after the unit's last co is
                // the first co of the next unit): the rest of this batch hides the scalar-load latency and only
                // this one request is outstanding at the next wait
                const float* __restrict__ apn =
                    bi + 1 < NB ? ap + RB : (last_co ? ap_next_unit : ap + (P.Mpad - (NB - 1) * RB));
                const f16v a_nxt = load_factors(apn);
                f16v g_nxt = a_nxt;
                if constexpr (IP == -2 || IP == -5) g_nxt = load_factors(apn + P.g_off);
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int q0 = RG; q0 < RB; q0 += RG) group(q0);
                a_cur = a_nxt;
                g_cur = g_nxt;
                ap = apn;
            }
            if (WITH_W) mine[(co - cur.co0) * kBwdSlab] = (gwp[0] + gwp[1]) + (gwp[2] + gwp[3]);
        }
        store_w((int)((u + 1) & 1), wstage);
        __syncthreads();  // every wave's partials of this unit are in its slot; the next unit's weights are in LDS
        if (WITH_W) {
            const int nco = cur.co1 - cur.co0;
            const float* __restrict__ buf = slots + (int)(u & 1) * NW * SLOT;
            for (int idx = threadIdx.x; idx < nco * kBwdSlab; idx += NT) {
                float v = 0.f;
                if constexpr (IP == -4) {
                    // idx >> 6 is the same co for the whole wave (64 divides every bound of this loop)
                    unsigned* hm = &hotmask[(int)(u & 1) * kBwdCoUnit + (idx >> 6)];
                    unsigned m = __builtin_amdgcn_readfirstlane(*hm);
                    if (m != 0) {
                        if ((idx & 63) == 0) *hm = 0u;  // clear for the unit after next
                        do {
                            v += buf[__builtin_ctz(m) * SLOT + idx];
                            m &= m - 1;
                        } while (m != 0);
                    }
                } else {
#pragma unroll
                    for (int wv_i = 0; wv_i < NW; wv_i++) v += buf[wv_i * SLOT + idx];
                }
                const int cl = idx >> 6, l = idx & 63;
                if (cur.ci0 + l < s.CIg) {
                    float* dst = GW + w_off(s, cur.g, cur.co0 + cl, cur.ci0 + l);
                    if (!P.gw_add) *dst = -v;
                    else atomicAdd(dst, -v);
                }
            }
        }
        cur = nxt;
    }
    flush_gx();
}

// Small batches (at most 32 rows; 33 to 64 rows take the two-wave configuration of the kernel above, which is a
// third faster there: no second row chunk adding into grad_weight).  The row-split kernel above would pad the rows to a whole workgroup and spend
// its time on the padding.  Here a workgroup owns 32 rows x one ci slab and its 16 waves split the co range
// instead: every wave keeps the same x rows, walks over its own co, and writes its grad_weight values straight from
// registers (complete for this row chunk).  The grad_x partials of the 16 waves are summed through LDS at the end and
// leave with one global atomic add per element and workgroup (adding them wave by wave would pile a hundred
// same-address atomics on every element).  The work is bound by streaming w and grad_w.
// Rows per chunk: 32, or 16 / 8 for batches that small (the arithmetic of the padded rows is the kernel's time there:
// one to eight rows at 5120 x 5120 took what 32 do).
constexpr int kBwdSmallRows = 32, kBwdSmallWaves = 16, kBwdSmallMaxM = 32;
inline int bwd_small_rows(int M) { return M <= 8 ? 8 : (M <= 16 ? 16 : kBwdSmallRows); }

template <int IP, bool WITH_W, int BT>
__global__ __launch_bounds__(64 * kBwdSmallWaves) void bwd_small_kernel(const float* __restrict__ X,
                                                                        const float* __restrict__ W,
                                                                        const float* __restrict__ AT,
                                                                        float* __restrict__ GX, float* __restrict__ GW,
                                                                        const BwdParams P, int cosplit, int cows) {
    constexpr int RB = BT < kBwdRowBatch ? BT : kBwdRowBatch, NB = BT / RB, RG = 4;
    static_assert(BT == 8 || BT == 16 || BT == 32, "row chunks of 8, 16 or 32");
    using FV = typename std::conditional<RB == 16, f16v, f8v>::type;  // one scalar load of RB factors
    auto load_fv = [](const float* p) __attribute__((always_inline)) -> FV {
        if constexpr (RB == 16) return load_factors(p);
        else return load_factors8(p);
    };
    const Geom& s = P.s;
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    if (P.gate != nullptr && ((P.gate[0] < P.gate_limit) != (P.gate_sense != 0))) return;
    const float thr = IP == -3 ? fast_exp2((fast_log2(P.gmax[0]) - 40.0f) / P.q) : 0.f;
    unsigned id = blockIdx.x;
    const int cs = (int)(id % (unsigned)cosplit);
    id /= (unsigned)cosplit;
    const int rc = (int)(id % (unsigned)P.nrc);
    id /= (unsigned)P.nrc;
    const int slab = (int)(id % (unsigned)P.nslab), g = (int)(id / (unsigned)P.nslab);
    const int co_begin = (cs * kBwdSmallWaves + wave) * cows, co_end = min(s.COg, co_begin + cows);
    const int ci = slab * kBwdSlab + lane;
    const bool ci_ok = ci < s.CIg;
    const int cic = min(ci, s.CIg - 1);  // clamped: unconditional loads, results of the excess lanes are dropped
    const int r0 = rc * BT;

    float xv[BT], gxa[BT];
#pragma unroll
    for (int i = 0; i < BT; i++) {
        const int m = min(r0 + i, s.M - 1);
        const int b = m / s.HW, hw = m - b * s.HW;
        xv[i] = X[x_off(s, b, g, cic, hw)];
        gxa[i] = 0.f;
    }
    const float* __restrict__ ap = AT + ((long)(g * s.COg + co_begin) * P.Mpad + r0);
    const float* __restrict__ wp = W + w_off(s, g, co_begin, cic);
    FV a_cur = load_fv(ap);
    FV g_cur = a_cur;
    if constexpr (IP == -2 || IP == -5) g_cur = load_fv(ap + P.g_off);
    float wnext = *wp;
    for (int co = co_begin; co < co_end; co++) {
        const float wv = wnext;
        const bool last_co = co + 1 == co_end;
        if (!last_co) wp += s.CIg;
        wnext = *wp;
        float gwp[RG] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int bi = 0; bi < NB; bi++) {
            float fa[RB], fg[RB];
#pragma unroll
            for (int r = 0; r < RB; r++) { fa[r] = a_cur[r]; fg[r] = g_cur[r]; }
            auto group = [&](int q0) {
                float ga[RG], gg[RG];
#pragma unroll
                for (int r = 0; r < RG; r++) { ga[r] = fa[q0 + r]; gg[r] = fg[q0 + r]; }
                bwd_terms<IP, WITH_W, RG>(&xv[bi * RB + q0], wv, ga, gg, P.q, thr, &gxa[bi * RB + q0], gwp);
            };
            group(0);
            __builtin_amdgcn_sched_barrier(0);
            // next batch: same co, next rows; or the next co (after the last co: a harmless re-read of this one)
            const float* __restrict__ apn = bi + 1 < NB ? ap + RB : (last_co ? ap - (NB - 1) * RB : ap + (P.Mpad - (NB - 1) * RB));
            const FV a_nxt = load_fv(apn);
            FV g_nxt = a_nxt;
            if constexpr (IP == -2 || IP == -5) g_nxt = load_fv(apn + P.g_off);
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int q0 = RG; q0 < RB; q0 += RG) group(q0);
            a_cur = a_nxt;
            g_cur = g_nxt;
            ap = apn;
        }
        if (WITH_W && ci_ok) {
            const float v = -((gwp[0] + gwp[1]) + (gwp[2] + gwp[3]));
            float* dst = GW + w_off(s, g, co, ci);
            if (!P.gw_add) *dst = v;
            else atomicAdd(dst, v);
        }
    }
    // ---- grad_x: sum over the waves, 16 rows at a time (16 waves x 16 rows x 64 lanes = 64 KB of LDS)
    constexpr int HR = BT < 16 ? BT : 16;
    __shared__ float red[kBwdSmallWaves * HR * kBwdSlab];
#pragma unroll
    for (int h = 0; h < BT / HR; h++) {
#pragma unroll
        for (int i = 0; i < HR; i++) red[(wave * HR + i) * kBwdSlab + lane] = gxa[h * HR + i];
        __syncthreads();
        if (wave < HR) {
            // thread -> (row = wave index, lane): one cell per thread
            float v = 0.f;
#pragma unroll
            for (int q = 0; q < kBwdSmallWaves; q++) v += red[(q * HR + wave) * kBwdSlab + lane];
            const int m = r0 + h * HR + wave;
            if (ci_ok && m < s.M) {
                const int b = m / s.HW, hw = m - b * s.HW;
                atomicAdd(GX + x_off(s, b, g, ci, hw), v);
            }
        }
        __syncthreads();
    }
}

struct BwdPtrs {
    const float* x;
    const float* w;
    const float* aT;
    float* gx;
    float* gw;  // nullptr: input gradient only
};

// rows per wave x waves per workgroup: 512 rows (one chunk at batch 512), 256 rows, 128 rows, and 64 rows for batches
// of 33 to 64 (six of those workgroups per compute unit).  Always 32 rows per
// wave (16 cost 26 % to 92 % more per row); two or four of the smaller workgroups share a compute unit, which the
// second launch bound (at least four waves per SIMD, i.e. at most 128 registers) makes possible.
constexpr int kBwdCfgRows[5] = {32, 32, 32, 0, 32};   // (index 3 is the small-batch kernel)
constexpr int kBwdCfgWaves[5] = {16, 8, 4, 0, 2};

// one explicit instantiation per exponent, spread over several translation units to compile in parallel
template <int IP>
int launch_bwd_ip(const BwdPtrs& a, const BwdParams& P, int cfg, int grid, hipStream_t st);

template <int IP>
int launch_bwd_ip_impl(const BwdPtrs& a, const BwdParams& P, int cfg, int grid, hipStream_t st) {
#define NDIST_BWD_LAUNCH(WITH_W, C)                                                                               \
    hipLaunchKernelGGL((bwd_fused_kernel<IP, WITH_W, kBwdCfgRows[C], kBwdCfgWaves[C]>), dim3(grid),               \
                       dim3(64 * kBwdCfgWaves[C]), 0, st, a.x, a.w, a.aT, a.gx, a.gw, P)
    KernelTimer timer(st);
    if (cfg == 3) {  // small batch: P was laid out for 32-row chunks by the caller
        const long wgs = (long)P.s.G * P.nslab * P.nrc;
        const int cus = device_info().num_cu;
        // split of the co range over workgroups: at least two workgroups per compute unit, at least 8 co per wave,
        // and among those the split whose last round of workgroups is the fullest (one workgroup fits a CU)
        const int most = P.s.COg / (kBwdSmallWaves * 8) > 1 ? P.s.COg / (kBwdSmallWaves * 8) : 1;
        int lo = (int)((2L * cus + wgs - 1) / wgs);
        lo = lo > most ? most : lo;
        int cosplit = lo;
        double best_eff = 0.0;
        for (int c = lo; c <= most && c <= 4 * lo; c++) {
            const double rounds = (double)wgs * c / cus;
            const double eff = rounds / (double)(long)(rounds + 0.999999);
            if (eff > best_eff + 1e-9) { best_eff = eff; cosplit = c; }
        }
        const int cows = ceil_div(P.s.COg, cosplit * kBwdSmallWaves);
        const dim3 g3((unsigned)(wgs * cosplit)), b3(64 * kBwdSmallWaves);
        const int bt = P.Mpad / P.nrc;  // rows per chunk, as the caller laid the factors out (bwd_small_rows)
#define NDIST_BWD_SMALL(WITH_W, BT_) \
    hipLaunchKernelGGL((bwd_small_kernel<IP, WITH_W, BT_>), g3, b3, 0, st, a.x, a.w, a.aT, a.gx, a.gw, P, cosplit, cows)
        if (a.gw != nullptr) {
            if (bt == 8) NDIST_BWD_SMALL(true, 8);
            else if (bt == 16) NDIST_BWD_SMALL(true, 16);
            else NDIST_BWD_SMALL(true, 32);
        } else {
            if (bt == 8) NDIST_BWD_SMALL(false, 8);
            else if (bt == 16) NDIST_BWD_SMALL(false, 16);
            else NDIST_BWD_SMALL(false, 32);
        }
#undef NDIST_BWD_SMALL
        return hip_failed(hipGetLastError()) ? 4 : 0;
    }
    if (a.gw != nullptr) {
        if (cfg == 0) NDIST_BWD_LAUNCH(true, 0);
        else if (cfg == 1) NDIST_BWD_LAUNCH(true, 1);
        else if (cfg == 2) NDIST_BWD_LAUNCH(true, 2);
        else NDIST_BWD_LAUNCH(true, 4);
    } else {
        if (cfg == 0) NDIST_BWD_LAUNCH(false, 0);
        else if (cfg == 1) NDIST_BWD_LAUNCH(false, 1);
        else if (cfg == 2) NDIST_BWD_LAUNCH(false, 2);
        else NDIST_BWD_LAUNCH(false, 4);
    }
#undef NDIST_BWD_LAUNCH
    return hip_failed(hipGetLastError()) ? 4 : 0;
}

}  // namespace ndist
