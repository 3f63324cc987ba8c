// Tiled forward skeleton shared by every forward kernel of the library.
//
// The forward of all operator variants has the shape of a matrix product with the multiply-accumulate replaced by
// another (reduction, pair-function) couple:  out[m, n] = REDUCE_k f(x[m, k], w[n, k]),  m = (b, hw), n = co,
// k = ci.  It runs on the FP32 vector ALU.  x comes in one of three layouts (a template parameter of the kernel):
// rows [B, C] with k contiguous, the unfolded convolution [B, C, HW] with the positions contiguous, or the images
// [B, C, H, W] of a convolutional layer themselves, in which case the loader extracts the patches (k = (c, i, j),
// m = (b, oh, ow), zeros outside the image) and the unfolded tensor never exists.
// One workgroup owns a BM x BN tile of outputs; each lane owns a
// TM x TN register micro-tile; x and w tiles are staged through LDS, k-major, so that a lane fetches its TM (TN)
// operands of one k with ds_read_b128; an XOR swizzle on the column index keeps both the transposing stores and the
// vector reads free of bank conflicts without padding.  A workgroup may split the k range of every stage over KS
// wave groups (2 waves per SIMD with the full-size micro-tile) and merges the partial results through LDS.
//
// The operator variants plug in as an `Op` policy: accumulator type, row function (one micro-tile row of TN outputs,
// two k at a time so that three-operand min/max instructions can be formed, written as stages of independent
// instructions), per-tile hook (arg-max bookkeeping), merge and finalisation.
#pragma once
#include <cstdlib>
#include <type_traits>

#include "ndist_common.h"

namespace ndist {

struct FwdParams {
    const float* x;    // input, or lower bound of the input box
    const float* x2;   // upper bound of the input box (interval variants), else unused
    const float* w;
    const float* aux;  // per output: caller-supplied normaliser (forward_with_max), or the seed of the running
                       // maximum of the skipping operator; else unused
    const float* aux2; // interval bounds with k-tile skipping: seed of the lower reduction (aux: of the upper one)
    float* out;        // output, or lower output bound
    float* out2;       // upper output bound
    int32_t* pos;      // per output: index of the winning k-tile (turned into the arg-max code by a rescan kernel)
    int32_t* pos2;
    Geom s;
    float p, inv_p;
    float thr, inv_thr;  // normalised sum with skipping: pairs below thr * (running maximum) are dropped
    int x_vec;  // rows of x may be fetched with aligned 16-byte loads
    int w_vec;
    int y_vec;  // outputs may be stored with aligned 16-byte stores
    int kt;     // k-tile length of the chosen configuration (set by the launcher; the rescan kernels need it)
    // split of the k range over workgroups (problems with too few output tiles to fill the device): workgroup z
    // handles group z / ksplit and the k range [z % ksplit * kchunk, +kchunk); with ksplit > 1 the raw accumulators go
    // to `partial` ([ksplit][words of Acc][total outputs]) and a merge kernel finishes the job
    int ksplit, kchunk;
    float* partial;
    long total;
    // optional gate: the kernel runs only when (gate[0] < gate_limit) == (gate_sense != 0); lets the launcher queue
    // two variants of an operator and have a device-side probe pick one without a host round trip
    const int* gate;
    int gate_limit, gate_sense;
    // Tile bounds (policies with TILE_BOUND): per row of x and per row of w, the largest magnitude inside every
    // 32-wide k-tile ([row][ntile32]).  |x - w| <= max|x| + max|w| lets a wave drop a whole k-tile of its step when
    // that bound stays below the thresholds of all its outputs.
    const float* tile_x;
    const float* tile_w;
    int ntile32;
    // implicit patch extraction: x (and x2) are images [B, C, H, W]; row m = (b, oh, ow) and k = (c, i, j) of the
    // distance "matrix" are mapped to image elements by the loader, taps outside the image read as zero -- the
    // values torch.nn.functional.unfold would have materialised.  s describes the unfolded problem.
    int implicit;
    PatchMap pm;
};

__device__ __forceinline__ bool gate_closed(const FwdParams& P) {
    return P.gate != nullptr && ((P.gate[0] < P.gate_limit) != (P.gate_sense != 0));
}

// policies that define TILE_BOUND = true are asked before every k-tile whether it can be skipped
template <class Op, class = void>
struct op_tile_bound : std::false_type {};
template <class Op>
struct op_tile_bound<Op, std::enable_if_t<Op::TILE_BOUND>> : std::true_type {};

// policies whose 256-thread configurations (two waves per SIMD, 256 registers) have room for a second operand set
// although their 1024-thread ones do not: `static constexpr bool PREFETCH_SMALL = true`
template <class Op, class = void>
struct op_prefetch_small : std::false_type {};
template <class Op>
struct op_prefetch_small<Op, std::enable_if_t<Op::PREFETCH_SMALL>> : std::true_type {};

template <int TM_, int TN_, int WM_, int WN_, int KS_, int KT_ = 32, int WAVES_ = 0>
struct TileCfg {
    static constexpr int TM = TM_, TN = TN_, WM = WM_, WN = WN_, KS = KS_;
    static constexpr int BM = TM * 8 * WM, BN = TN * 8 * WN;
    static constexpr int NTG = kWave * WM * WN;  // threads of one k-group
    static constexpr int NT = NTG * KS;
    static constexpr int KT = KT_;               // k per group per stage == arg-max tile granularity
    static constexpr int KTOT = KT * KS;
    static constexpr int LDM = round_up(BM, 64), LDN = round_up(BN, 64);
    // waves per SIMD the register allocation must leave room for: four for the 1024-thread workgroups (one per
    // compute unit), two for the smaller ones, unless the configuration asks for more (two 1024-thread workgroups
    // per compute unit: eight)
    static constexpr int WAVES = WAVES_ > 0 ? WAVES_ : (NT >= 1024 ? 4 : 2);
};

// column of micro-tile slot j for lane index t (0..7) inside a wave-tile that is 8*T wide:
// the first 4*(T/4) slots are groups of four consecutive columns, the rest are strided by 8
template <int T>
__device__ __forceinline__ int micro_col(int j, int t) {
    constexpr int Q = T / 4;
    return j < 4 * Q ? (j / 4) * 32 + t * 4 + (j % 4) : Q * 32 + (j - 4 * Q) * 8 + t;
}

template <int T>
__device__ __forceinline__ void read_micro(const float* __restrict__ row, int base, int t, int sw, float (&v)[T]) {
    constexpr int Q = T / 4;
#pragma unroll
    for (int q = 0; q < Q; q++) {
        const float4 f = *reinterpret_cast<const float4*>(row + ((base + q * 32 + t * 4) ^ sw));
        v[4 * q + 0] = f.x; v[4 * q + 1] = f.y; v[4 * q + 2] = f.z; v[4 * q + 3] = f.w;
    }
#pragma unroll
    for (int r = 0; r < T - 4 * Q; r++) v[4 * Q + r] = row[(base + Q * 32 + r * 8 + t) ^ sw];
}

__device__ __forceinline__ float4 load4_guarded(const float* __restrict__ src, int k, int K, bool row_ok, bool vec) {
    float4 r = make_float4(0.f, 0.f, 0.f, 0.f);
    if (row_ok) {
        if (vec && k + 3 < K) {
            r = *reinterpret_cast<const float4*>(src + k);
        } else {
            if (k + 0 < K) r.x = src[k + 0];
            if (k + 1 < K) r.y = src[k + 1];
            if (k + 2 < K) r.z = src[k + 2];
            if (k + 3 < K) r.w = src[k + 3];
        }
    }
    return r;
}

// At least two waves per SIMD: a 256-thread configuration must leave room for a second workgroup on the compute unit
// (a register count just above 256 would halve the occupancy and cost far more than the few spills it avoids).
// LAYOUT: 0 = [B, C] rows (HW == 1), 1 = [B, C, HW] with positions contiguous, 2 = images with implicit patches
template <class Op, class Cfg, int LAYOUT>
__global__ __launch_bounds__(Cfg::NT) __attribute__((amdgpu_waves_per_eu(Cfg::WAVES)))
void fwd_tile_kernel(const FwdParams P) {
    constexpr int TM = Cfg::TM, TN = Cfg::TN, WN = Cfg::WN, WM = Cfg::WM, BM = Cfg::BM, BN = Cfg::BN;
    constexpr int KT = Cfg::KT, KS = Cfg::KS, KTOT = Cfg::KTOT, NT = Cfg::NT, NTG = Cfg::NTG;
    constexpr int LDM = Cfg::LDM, LDN = Cfg::LDN, NX = Op::NX;
    constexpr int XS = KTOT * LDM, WS = KTOT * LDN, STAGE = NX * XS + WS;
    using Acc = typename Op::Acc;
    constexpr int NF = sizeof(Acc) / 4;
    static_assert(2 * STAGE >= (KS - 1) * NTG * NF * TN, "merge buffer must fit in the tile buffers");
    __shared__ __attribute__((aligned(16))) float smem[2 * STAGE];
    constexpr bool HAS_HW = LAYOUT != 0, IMPLICIT = LAYOUT == 2;
    // tile bounds of the two stages: per k-group the maxima of the BM rows of x, then of the BN rows of w
    constexpr bool BOUNDS = op_tile_bound<Op>::value;
    constexpr int NBND = KS * (LDM + LDN), BP = BOUNDS ? ceil_div(NBND, NT) : 1;
    static_assert(!BOUNDS || KT == 32, "tile bounds are kept per 32 k");
    // Bounds run three stages ahead of the data in a ring of four, so that the workgroup can vote on a stage before
    // its loads would have to be issued: need[j] says whether any wave still wants the stage in ring slot j.
    constexpr int RING = 4;
    __shared__ __attribute__((aligned(16))) float bnd[BOUNDS ? RING * NBND : 4];
    __shared__ int need[RING];

    if (gate_closed(P)) return;
    const Geom& s = P.s;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int kg = wave / (WM * WN), wsub = wave % (WM * WN), wm = wsub / WN, wn = wsub % WN;
    const int tx = lane & 7, ty = lane >> 3;
    const int im = HAS_HW ? tx : ty, in = HAS_HW ? ty : tx;  // the contiguous output axis runs along tx
    const int g = blockIdx.z / P.ksplit, sp = blockIdx.z % P.ksplit;
    // Workgroups are handed to the 8 XCDs (each with its own L2) round-robin by linear id.  The tiles are renumbered
    // so that an XCD gets a contiguous run of them, ordered row tile fastest: the workgroups of one XCD then share a
    // few column tiles of w and all row tiles of x, instead of every XCD streaming most of w through its L2.
    int mt = blockIdx.x, nt = blockIdx.y;
    {
        constexpr int kXcd = 8;
        const int ntm = gridDim.x, nwg = gridDim.x * gridDim.y;
        if (nwg >= 2 * kXcd) {
            const int id = blockIdx.y * ntm + blockIdx.x;
            const int xcd = id % kXcd, slot = id / kXcd, q = nwg / kXcd, r = nwg % kXcd;
            const int v = xcd * q + min(xcd, r) + slot;
            mt = v % ntm;
            nt = v / ntm;
        }
    }
    const int m0 = mt * BM, n0 = nt * BN;
    const int K = s.CIg;                       // row stride of x and w
    const int kb = sp * P.kchunk;              // this workgroup's k range: [kb, KE)
    const int KE = min(K, kb + P.kchunk);

    // ---- staging descriptors -------------------------------------------------------------------------
    // row-major sources (k contiguous): a thread fetches 4 consecutive k of one row per pass
    constexpr int KQ = KTOT / 4, RP = NT / KQ;
    constexpr int WP = ceil_div(BN, RP);
    constexpr int XP_FC = ceil_div(BM, RP);
    // k-major source (conv layout, m contiguous): a thread fetches 4 consecutive m of one k per pass
    constexpr int MQ = BM / 4, KP = NT / MQ;
    constexpr int XP_HW = ceil_div(KTOT, KP);
    constexpr int XP = HAS_HW ? XP_HW : XP_FC;
    static_assert(NT % KQ == 0 && NT % MQ == 0, "tile shape");
    // XOR swizzle of the column index by the 4-k chunk the row belongs to.  The transposing store of a wave covers
    // KQ chunks x (64 / KQ) consecutive rows: shifting the chunk index by log2(64 / KQ) spreads them over all 64
    // banks; any shift >= 2 keeps four consecutive columns together for the 16-byte operand reads.
    static_assert(KQ == 8 || KQ == 16, "swizzle is laid out for 32 or 64 k per stage");
    constexpr int SWS = KQ == 16 ? 2 : 3, SWM = KQ - 1;
    auto swz = [](int k_local) { return ((k_local >> 2) & SWM) << SWS; };

    const int kq = tid % KQ, rr = tid / KQ;
    const int mq = tid % MQ, kr = tid / MQ;
    const float* __restrict__ wbase = P.w + (long)g * s.COg * K;
    // conv layout: the four rows m .. m+3 this thread stages (same image when the vector path is allowed)
    int hb = 0, hhw = 0;
    int cih = 0, ciw = 0;  // implicit patches: top-left tap of the first of the four positions
    if (HAS_HW) {
        const int m = m0 + 4 * mq;
        hb = m / s.HW;
        hhw = m - hb * s.HW;
        if (IMPLICIT) patch_origin(P.pm, hhw, cih, ciw);
    }

    float4 xr[NX][XP], wr[WP];
    float br[BP];  // tile bounds on their way to LDS

    auto fetch_x = [&](const float* __restrict__ xp, float4 (&dst)[XP], int kbase) __attribute__((always_inline)) {
        if (!HAS_HW) {
#pragma unroll
            for (int i = 0; i < XP; i++) {
                const int row = rr + i * RP, m = m0 + row;
                const bool ok = (BM % RP == 0 || row < BM) && m < s.M;
                const float* src = xp + ((long)m * s.G + g) * K;
                dst[i] = load4_guarded(src, kbase + 4 * kq, KE, ok, P.x_vec);
            }
        } else {
#pragma unroll
            for (int i = 0; i < XP; i++) {
                const int kl = kr + i * KP, k = kbase + kl;
                const int m = m0 + 4 * mq;
                float4 r = make_float4(0.f, 0.f, 0.f, 0.f);
                if (IMPLICIT) {
                    if ((KTOT % KP == 0 || kl < KTOT) && k < KE) {
                        const PatchTap tp = patch_tap(P.pm, g, k);
                        if (P.x_vec) {  // the four positions share one output row (OW % 4 == 0)
                            if (m < s.M) r = patch_row4(xp, P.pm, hb, tp, cih, ciw);
                        } else {
                            auto tap_at = [&](int mj) __attribute__((always_inline)) {
                                return mj < s.M ? patch_elem(xp, P.pm, mj / s.HW, tp, mj % s.HW) : 0.f;
                            };
                            r = make_float4(tap_at(m), tap_at(m + 1), tap_at(m + 2), tap_at(m + 3));
                        }
                    }
                } else if ((KTOT % KP == 0 || kl < KTOT) && k < KE) {
                    if (P.x_vec && m + 3 < s.M) {
                        r = *reinterpret_cast<const float4*>(xp + (((long)hb * s.G + g) * K + k) * s.HW + hhw);
                    } else {
                        float t[4];
#pragma unroll
                        for (int j = 0; j < 4; j++) {
                            const int mj = m + j;
                            t[j] = 0.f;
                            if (mj < s.M) {
                                const int b = mj / s.HW, hw = mj - b * s.HW;
                                t[j] = xp[(((long)b * s.G + g) * K + k) * s.HW + hw];
                            }
                        }
                        r = make_float4(t[0], t[1], t[2], t[3]);
                    }
                }
                dst[i] = r;
            }
        }
    };
    auto fetch_bounds = [&](int kbase) __attribute__((always_inline)) {
#pragma unroll
        for (int i = 0; i < BP; i++) {
            const int e = tid + i * NT, grp = e / (LDM + LDN), c = e - grp * (LDM + LDN);
            const int t32 = kbase / 32 + grp;
            float v = P.tile_x != nullptr ? 0.f : __builtin_inff();  // no bounds supplied: nothing is skipped
            if (P.tile_x != nullptr && e < NBND && t32 < P.ntile32) {
                if (c < LDM) {
                    const int m = m0 + c;
                    if (c < BM && m < s.M) v = P.tile_x[((long)m * s.G + g) * P.ntile32 + t32];
                } else {
                    const int n = n0 + c - LDM;
                    if (c - LDM < BN && n < s.COg) v = P.tile_w[((long)g * s.COg + n) * P.ntile32 + t32];
                }
            }
            br[i] = v;
        }
    };
    auto put_bounds = [&](int slot) __attribute__((always_inline)) {
        float* bd = bnd + slot * NBND;
#pragma unroll
        for (int i = 0; i < BP; i++)
            if (tid + i * NT < NBND) bd[tid + i * NT] = br[i];
    };
    auto fetch = [&](int kbase) __attribute__((always_inline)) {
        fetch_x(P.x, xr[0], kbase);
        if (NX == 2) fetch_x(P.x2, xr[NX - 1], kbase);
#pragma unroll
        for (int i = 0; i < WP; i++) {
            const int row = rr + i * RP, n = n0 + row;
            const bool ok = (BN % RP == 0 || row < BN) && n < s.COg;
            wr[i] = load4_guarded(wbase + (long)n * K, kbase + 4 * kq, KE, ok, P.w_vec);
        }
    };
    auto put = [&](float* __restrict__ buf) __attribute__((always_inline)) {
        float* xs = buf;
        float* ws = buf + NX * XS;
        if (NX == 2) {
            // an inverted box collapses to its midpoint (reference: core/cuda/bound_inf_dist_cuda.cu:63)
#pragma unroll
            for (int i = 0; i < XP; i++) {
                float* a = reinterpret_cast<float*>(&xr[0][i]);
                float* c = reinterpret_cast<float*>(&xr[NX - 1][i]);
#pragma unroll
                for (int j = 0; j < 4; j++)
                    if (a[j] > c[j]) a[j] = c[j] = (a[j] + c[j]) * 0.5f;
            }
        }
#pragma unroll
        for (int a = 0; a < NX; a++) {
            float* dstx = xs + a * XS;
            if (!HAS_HW) {
                const int sw = swz(4 * kq);
#pragma unroll
                for (int i = 0; i < XP; i++) {
                    const int row = rr + i * RP;
                    if (BM % RP == 0 || row < BM) {
                        const int c = row ^ sw;
                        dstx[(4 * kq + 0) * LDM + c] = xr[a][i].x;
                        dstx[(4 * kq + 1) * LDM + c] = xr[a][i].y;
                        dstx[(4 * kq + 2) * LDM + c] = xr[a][i].z;
                        dstx[(4 * kq + 3) * LDM + c] = xr[a][i].w;
                    }
                }
            } else {
#pragma unroll
                for (int i = 0; i < XP; i++) {
                    const int kl = kr + i * KP;
                    if (KTOT % KP == 0 || kl < KTOT) {
                        const int sw = swz(kl);
                        *reinterpret_cast<float4*>(dstx + kl * LDM + ((4 * mq) ^ sw)) = xr[a][i];
                    }
                }
            }
        }
        {
            const int sw = swz(4 * kq);
#pragma unroll
            for (int i = 0; i < WP; i++) {
                const int row = rr + i * RP;
                if (BN % RP == 0 || row < BN) {
                    const int c = row ^ sw;
                    ws[(4 * kq + 0) * LDN + c] = wr[i].x;
                    ws[(4 * kq + 1) * LDN + c] = wr[i].y;
                    ws[(4 * kq + 2) * LDN + c] = wr[i].z;
                    ws[(4 * kq + 3) * LDN + c] = wr[i].w;
                }
            }
        }
    };

    // ---- accumulators --------------------------------------------------------------------------------
    Acc acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; i++)
#pragma unroll
        for (int j = 0; j < TN; j++) {
            const int m = m0 + wm * TM * 8 + micro_col<TM>(i, im);
            const int n = n0 + wn * TN * 8 + micro_col<TN>(j, in);
            Op::init(acc[i][j], P, kg + sp, m, n, g);  // the once-only terms belong to k-group 0 of split 0
        }

    const int ntiles = ceil_div(KE - kb, KTOT), tile0 = kb / KTOT;
    // BOUNDS: can this wave drop stage t (its bounds are in ring slot t % RING)?
    auto wave_skips = [&](int t) __attribute__((always_inline)) -> bool {
        if constexpr (BOUNDS) {
            const float* bd = bnd + (t % RING) * NBND + kg * (LDM + LDN);
            float bx[TM], bw[TN];
            read_micro<TM>(bd, wm * TM * 8, im, 0, bx);
            read_micro<TN>(bd + LDM, wn * TN * 8, in, 0, bw);
            return Op::template tile_skip<TM, TN>(acc, bx, bw);
        } else {
            return false;
        }
    };
    auto compute_tile = [&](int t, bool skip_tile) __attribute__((always_inline)) {
        const float* buf = smem + (t & 1) * STAGE;
        const float* xs = buf + kg * KT * LDM;
        const float* ws = buf + NX * XS + kg * KT * LDN;
#pragma unroll
        for (int ph = 0; ph < Op::PHASES; ph++) {
            if (BOUNDS && skip_tile) break;  // wave-uniform: nothing in this k-tile can count for this wave
            // operands of two consecutive k per step, double-buffered in registers: the LDS reads of step i+1 are
            // in flight while step i is computed
            float a0[2][TM], a1[2][TM], c0[2][TM], c1[2][TM], b0[2][TN], b1[2][TN];
            auto read_step = [&](int kk, int slot) {
                const int sw = swz(kg * KT + kk);
                read_micro<TM>(xs + kk * LDM, wm * TM * 8, im, sw, a0[slot]);
                read_micro<TM>(xs + (kk + 1) * LDM, wm * TM * 8, im, sw, a1[slot]);
                if (NX == 2) {
                    read_micro<TM>(xs + XS + kk * LDM, wm * TM * 8, im, sw, c0[slot]);
                    read_micro<TM>(xs + XS + (kk + 1) * LDM, wm * TM * 8, im, sw, c1[slot]);
                }
                read_micro<TN>(ws + kk * LDN, wn * TN * 8, in, sw, b0[slot]);
                read_micro<TN>(ws + (kk + 1) * LDN, wn * TN * 8, in, sw, b1[slot]);
            };
            auto compute_step = [&](int slot) {
                // one micro-tile row (TN outputs x 2 k) at a time: the policy lays its arithmetic out in stages of
                // independent instructions, because back-to-back dependent vector instructions stall the wave
#pragma unroll
                for (int i = 0; i < TM; i++)
                    Op::template row2<TN>(acc[i], P, ph, a0[slot][i], NX == 2 ? c0[slot][i] : 0.f, b0[slot], a1[slot][i],
                                          NX == 2 ? c1[slot][i] : 0.f, b1[slot]);
            };
            static_assert(KT % 4 == 0, "two steps of two k per iteration");
            if constexpr ((Op::PREFETCH && NT <= 512) || (op_prefetch_small<Op>::value && NT <= 256)) {
                // (the last iteration is peeled: a read under a condition at the end of the loop body makes the
                // compiler carry both operand sets through copies, one v_mov per register and iteration)
                read_step(0, 0);
#pragma unroll 1
                for (int kk = 0; kk < KT - 4; kk += 4) {
                    read_step(kk + 2, 1);
                    compute_step(0);
                    read_step(kk + 4, 0);
                    compute_step(1);
                }
                read_step(KT - 2, 1);
                compute_step(0);
                compute_step(1);
            } else {  // register-hungry accumulators: no room for a second operand set
#pragma unroll 2
                for (int kk = 0; kk < KT; kk += 2) {
                    read_step(kk, 0);
                    compute_step(0);
                }
            }
#pragma unroll
            for (int i = 0; i < TM; i++)
#pragma unroll
                for (int j = 0; j < TN; j++) Op::phase_end(acc[i][j], P, ph, (tile0 + t) * KS + kg);
        }
    };
    if constexpr (!BOUNDS) {
        fetch(kb);
        put(smem);
        __syncthreads();
        for (int t = 0; t < ntiles; t++) {
            if (t + 1 < ntiles) fetch(kb + (t + 1) * KTOT);
            compute_tile(t, false);
            if (t + 1 < ntiles) put(smem + ((t + 1) & 1) * STAGE);
            __syncthreads();
        }
    } else {
        // Stages the whole workgroup can drop are not even loaded.  The thresholds of the policy only tighten, so a
        // stage that no wave wants now is wanted by none later: during stage t every wave looks at the bounds of
        // stage t + 2 and raises need[] if it cannot drop it; the barrier that ends stage t publishes the flags, and
        // stage t + 1 decides on them whether to issue the loads of stage t + 2.  The first two stages are always
        // loaded.  Ring slots: bounds of stage t + 3 are fetched during stage t into the slot of stage t - 1, whose
        // last reader ran before the previous barrier; the flag of that slot is cleared at the same time, one
        // barrier before the votes of stage t + 1 write it.  A wave's own decision on a stage is the one it took in the
        // vote, two stages earlier (skip0 / skip1 hold the decisions on the current and the next stage).
#pragma unroll 1
        for (int t = 0; t < 3 && t < ntiles; t++) {
            fetch_bounds(kb + t * KTOT);
            put_bounds(t);
        }
        if (tid < RING) need[tid] = tid < 2 ? 1 : 0;
        fetch(kb);
        put(smem);
        __syncthreads();
        bool skip0 = wave_skips(0), skip1 = ntiles > 1 ? wave_skips(1) : true;
        for (int t = 0; t < ntiles; t++) {
            const bool cur = __builtin_amdgcn_readfirstlane(need[t % RING]) != 0;
            const bool nxt = t + 1 < ntiles && __builtin_amdgcn_readfirstlane(need[(t + 1) % RING]) != 0;
            if (nxt) fetch(kb + (t + 1) * KTOT);
            if (t + 3 < ntiles) fetch_bounds(kb + (t + 3) * KTOT);
            if (cur) compute_tile(t, skip0);
            const bool skip2 = t + 2 < ntiles ? wave_skips(t + 2) : true;
            if (!skip2 && lane == 0) need[(t + 2) % RING] = 1;
            skip0 = skip1;
            skip1 = skip2;
            if (tid == 0) need[(t + 3) % RING] = 0;
            if (nxt) put(smem + ((t + 1) & 1) * STAGE);
            if (t + 3 < ntiles) put_bounds((t + 3) % RING);
            __syncthreads();
        }
    }

    // ---- merge the k-groups (one micro-tile row at a time, through the now idle tile buffers) ---------
    if (KS > 1) {
        const int tig = tid % NTG;
#pragma unroll
        for (int i = 0; i < TM; i++) {
            if (kg > 0) {
#pragma unroll
                for (int j = 0; j < TN; j++) {
                    float f[NF];
                    __builtin_memcpy(f, &acc[i][j], sizeof(Acc));
#pragma unroll
                    for (int q = 0; q < NF; q++) smem[(((kg - 1) * TN + j) * NF + q) * NTG + tig] = f[q];
                }
            }
            __syncthreads();
            if (kg == 0) {
#pragma unroll
                for (int o = 1; o < KS; o++)
#pragma unroll
                    for (int j = 0; j < TN; j++) {
                        float f[NF];
#pragma unroll
                        for (int q = 0; q < NF; q++) f[q] = smem[(((o - 1) * TN + j) * NF + q) * NTG + tig];
                        Acc other;
                        __builtin_memcpy(&other, f, sizeof(Acc));
                        Op::merge(acc[i][j], other, P);
                    }
            }
            __syncthreads();
        }
        if (kg > 0) return;
    }

    // ---- k range split over workgroups: raw accumulators to scratch, finished by fwd_merge_kernel --------
    if (P.ksplit > 1) {
#pragma unroll
        for (int i = 0; i < TM; i++)
#pragma unroll
            for (int j = 0; j < TN; j++) {
                const int m = m0 + wm * TM * 8 + micro_col<TM>(i, im);
                const int n = n0 + wn * TN * 8 + micro_col<TN>(j, in);
                if (m < s.M && n < s.COg) {
                    const int b = HAS_HW ? m / s.HW : m, hw = HAS_HW ? m - b * s.HW : 0;
                    float f[NF];
                    __builtin_memcpy(f, &acc[i][j], sizeof(Acc));
#pragma unroll
                    for (int q = 0; q < NF; q++) P.partial[((long)sp * NF + q) * P.total + y_off(s, b, g, n, hw)] = f[q];
                }
            }
        return;
    }

    // ---- finalise and store --------------------------------------------------------------------------
    constexpr int NOF = Op::NOF, NOI = Op::NOI;
    float* fo[2] = {P.out, P.out2};
    int32_t* io[2] = {P.pos, P.pos2};
    // micro-tile slots 0..3 of the contiguous axis are four consecutive outputs: store them as one vector
    constexpr int TC = HAS_HW ? TM : TN;  // slots along the contiguous output axis
    constexpr int TR = HAS_HW ? TN : TM;
#pragma unroll
    for (int r = 0; r < TR; r++) {
#pragma unroll
        for (int c4 = 0; c4 < TC; c4 += 4) {
            const bool vecgrp = c4 + 3 < 4 * (TC / 4);
            float fv[4][NOF > 0 ? NOF : 1];
            int iv[4][NOI > 0 ? NOI : 1];
            long off[4];
            bool ok[4];
#pragma unroll
            for (int c = 0; c < 4; c++) {
                ok[c] = false;
                off[c] = 0;
                if (c4 + c < TC) {
                    const int i = HAS_HW ? c4 + c : r, j = HAS_HW ? r : c4 + c;
                    const int m = m0 + wm * TM * 8 + micro_col<TM>(i, im);
                    const int n = n0 + wn * TN * 8 + micro_col<TN>(j, in);
                    Op::finalize(acc[i][j], P, fv[c], iv[c]);
                    ok[c] = m < s.M && n < s.COg;
                    if (ok[c]) {
                        const int b = HAS_HW ? m / s.HW : m, hw = HAS_HW ? m - b * s.HW : 0;
                        off[c] = y_off(s, b, g, n, hw);
                    }
                }
            }
            if (vecgrp && P.y_vec && ok[0] && ok[3]) {
#pragma unroll
                for (int q = 0; q < NOF; q++)
                    *reinterpret_cast<float4*>(fo[q] + off[0]) = make_float4(fv[0][q], fv[1][q], fv[2][q], fv[3][q]);
#pragma unroll
                for (int q = 0; q < NOI; q++)
                    *reinterpret_cast<int4*>(io[q] + off[0]) = make_int4(iv[0][q], iv[1][q], iv[2][q], iv[3][q]);
            } else {
#pragma unroll
                for (int c = 0; c < 4; c++)
                    if (ok[c]) {
#pragma unroll
                        for (int q = 0; q < NOF; q++) fo[q][off[c]] = fv[c][q];
#pragma unroll
                        for (int q = 0; q < NOI; q++) io[q][off[c]] = iv[c][q];
                    }
            }
        }
    }
}

// ---- host side: configuration choice and launch -------------------------------------------------------

using CfgBig = TileCfg<8, 8, 2, 2, 1>;    // 128 x 128, 256 threads
using CfgWide = TileCfg<8, 5, 2, 2, 2>;   // 128 x 80, 512 threads, k split in two: 256 tiles at 512 x 5120
using CfgWide4 = TileCfg<8, 5, 2, 2, 4, 16>;  // same tile, 1024 threads, k split in four: 4 waves per SIMD
using CfgWideT = TileCfg<4, 5, 4, 2, 2, 32>;  // same tile, 1024 threads, half-height micro-tile: room for arg-max state
using CfgBoundN = TileCfg<4, 5, 4, 2, 2, 16>;  // 128 x 80 for two input arrays (interval bounds), 1024 threads:
                                               // half-height micro-tile, k split in two, 32 k per stage
using CfgBoundT = TileCfg<4, 5, 4, 2, 1, 32>;  // 128 x 80, half-height micro-tile: six registers of state per output
using CfgMid = TileCfg<8, 4, 2, 2, 1>;    // 128 x 64, 256 threads
using CfgSmall = TileCfg<4, 4, 2, 2, 1>;  // 64 x 64, 256 threads
// the same held to 128 registers (four waves per SIMD): the arg-max kernel's three registers per output allow it at
// the price of a few spills, and it measures 1 - 8 % faster in the layouts with positions
using CfgSmall4 = TileCfg<4, 4, 2, 2, 1, 32, 4>;
// batches of at most 32 / 16 rows: a 64-row tile would spend half or more of its work on padding (finite-p forward at
// 5120 x 5120: 0.166 -> 0.108 ms at 32 rows, 0.162 -> 0.068 ms at 8 and 16)
using CfgLow32 = TileCfg<4, 4, 1, 4, 1>;  // 32 x 128, 256 threads
using CfgLow16 = TileCfg<2, 8, 1, 4, 1>;  // 16 x 256, 256 threads
// 33 to 64 rows: the 1024-thread tile at half height (64 x 80): four waves per SIMD from one workgroup per compute
// unit, where the 256-thread 64 x 64 tiles leave the SIMDs with two (p = 8 at 64 x 5120 x 5120: 0.176 -> 0.160 ms)
using CfgWide4H = TileCfg<4, 5, 2, 2, 4, 16>;
// the same 64 x 80 tile on 8 k per wave group and stage (48 KB of LDS) within 64 registers: two 1024-thread workgroups
// per compute unit, eight waves per SIMD (measurement aid: only ever chosen through NORM_DIST_TILE_CFG)
using CfgOcc8 = TileCfg<4, 5, 2, 2, 4, 8, 8>;
using CfgOcc8W = TileCfg<4, 5, 4, 2, 2, 16, 8>;  // 128 x 80, 16 k per wave group and stage (64 KB of LDS), likewise

// Second step of a split k range: merges the partial accumulators of one output in split order, finalises, stores.
template <class Op>
__global__ __launch_bounds__(256) void fwd_merge_kernel(const FwdParams P) {
    using Acc = typename Op::Acc;
    constexpr int NF = sizeof(Acc) / 4, NOF = Op::NOF, NOI = Op::NOI;
    const long o = (long)blockIdx.x * 256 + threadIdx.x;
    if (o >= P.total || gate_closed(P)) return;
    auto load = [&](int sp) {
        float f[NF];
#pragma unroll
        for (int q = 0; q < NF; q++) f[q] = P.partial[((long)sp * NF + q) * P.total + o];
        Acc a;
        __builtin_memcpy(&a, f, sizeof(Acc));
        return a;
    };
    Acc a = load(0);
    for (int sp = 1; sp < P.ksplit; sp++) Op::merge(a, load(sp), P);
    float fv[NOF > 0 ? NOF : 1];
    int iv[NOI > 0 ? NOI : 1];
    Op::finalize(a, P, fv, iv);
    float* fo[2] = {P.out, P.out2};
    int32_t* io[2] = {P.pos, P.pos2};
#pragma unroll
    for (int q = 0; q < NOF; q++) fo[q][o] = fv[q];
#pragma unroll
    for (int q = 0; q < NOI; q++) io[q][o] = iv[q];
}

template <class Op, class Cfg, bool CONV>
int launch_cfg(FwdParams P, int ksplit, hipStream_t st) {
    const Geom& s = P.s;
    using Acc = typename Op::Acc;
    P.kt = Cfg::KT;
    P.ksplit = ksplit;
    P.kchunk = ksplit > 1 ? round_up(ceil_div(s.CIg, ksplit), Cfg::KTOT) : s.CIg;
    P.total = (long)s.M * s.COg * s.G;
    P.partial = nullptr;
    if (P.implicit && !CONV) return 2;
    KernelTimer timer(st);
    if (ksplit > 1) {
        NDIST_HIP_TRY(scratch_alloc((void**)&P.partial, (size_t)ksplit * sizeof(Acc) * P.total, st));
    }
    dim3 grid(ceil_div(s.M, Cfg::BM), ceil_div(s.COg, Cfg::BN), s.G * ksplit);
    if (P.implicit) {
        if constexpr (CONV) hipLaunchKernelGGL((fwd_tile_kernel<Op, Cfg, 2>), grid, dim3(Cfg::NT), 0, st, P);
    } else if (s.HW == 1) {
        hipLaunchKernelGGL((fwd_tile_kernel<Op, Cfg, 0>), grid, dim3(Cfg::NT), 0, st, P);
    } else {
        hipLaunchKernelGGL((fwd_tile_kernel<Op, Cfg, 1>), grid, dim3(Cfg::NT), 0, st, P);
    }
    int rc = hip_failed(hipGetLastError()) ? 4 : 0;
    if (ksplit > 1) {
        if (!rc) {
            hipLaunchKernelGGL((fwd_merge_kernel<Op>), dim3((unsigned)((P.total + 255) / 256)), dim3(256), 0, st, P);
            rc = hip_failed(hipGetLastError()) ? 4 : 0;
        }
        if (hip_failed(scratch_free(P.partial, st)) && !rc) rc = 4;
    }
    return rc;
}

// Split of the k range a configuration would use.  256-thread workgroups (one wave per SIMD each; several share a
// compute unit): none while the tiles fill the device twice, otherwise enough parts for about two workgroups per
// compute unit.  Larger workgroups (one per compute unit at a time, all tiles cost the same, so the device works
// in rounds): the split that leaves the fewest idle compute units in the last round, e.g. 192 tiles on 256 units
// run as 768 quarter tiles in three full rounds instead of 384 half tiles in two rounds, the second half empty.
// Each part is at least four stages long.  Every part costs the trip of its partial results through memory:
// `part_cost` is that trip relative to the whole kernel (see split_part_cost), 0.3 % to 3 % per part at k = 5120.
template <class Cfg>
int tile_ksplit(const Geom& s, int cus, double part_cost) {
    const long tiles = (long)ceil_div(s.M, Cfg::BM) * ceil_div(s.COg, Cfg::BN) * s.G;
    int by_k = ceil_div(s.CIg, Cfg::KTOT) / 4;
    by_k = by_k < 1 ? 1 : (by_k > 64 ? 64 : by_k);
    if (Cfg::NT <= 256) {
        if (tiles >= 2L * cus) return 1;
        const int by_cu = (int)(2L * cus / tiles);
        const int ks = by_k < by_cu ? by_k : by_cu;
        return ks < 1 ? 1 : ks;
    }
    int best = 1;
    double best_cost = 0.0;
    for (int ks = 1; ks <= by_k; ks++) {
        const long rounds = (tiles * ks + cus - 1) / cus;
        if (ks > 1 && rounds > 64) break;  // many rounds: the last one no longer matters
        const double cost = (double)rounds / ks * (ks > 1 ? 1.01 + part_cost * ks : 1.0);
        if (ks == 1 || cost < best_cost - 1e-9) { best_cost = cost; best = ks; }
    }
    return best;
}

// One more part of a split k range writes and reads sizeof(Acc) bytes per output; relative to the operator's own
// work on the output's k pairs (Op::COST issue cycles per pair and wave; p = 8: 10.5 cycles = 68 fs per pair on the
// whole device, memory at about 3 TB/s for this pattern) that is sizeof(Acc) * 100 / (k * COST).
template <class Op>
double split_part_cost(const Geom& s) {
    return (double)sizeof(typename Op::Acc) * 100.0 / ((double)s.CIg * Op::COST);
}

// Estimated time of covering the problem with the tiles of one configuration: tiles the busiest compute unit
// runs, times the tile area (padding at ragged edges is paid for, idle compute units too), times a factor for
// the LDS traffic of the micro-tile shape, divided by the split of the k range.  A 256-thread workgroup alone on its
// compute unit (one wave per SIMD, nothing to hide latencies behind) runs at little more than half its speed.
// Measured on top of that: per pair the 256-thread tiles are 7 % to 15 % slower than the 512- and 1024-thread ones.
// Policies with several registers of state per output (arg-max bookkeeping, two reductions of the interval bounds):
// `static constexpr bool HEAVY = true`.  Their 128 x 64 tiles run two waves per SIMD where the 64 x 64 ones run
// three, and measure 0 - 20 % slower per pair (6 % on the 3 x 3 convolution with 128 channels).
template <class Op, class = void>
struct op_heavy : std::false_type {};
template <class Op>
struct op_heavy<Op, std::enable_if_t<Op::HEAVY>> : std::true_type {};

template <class Op, class Cfg>
double tile_cost(const Geom& s, int cus, double part_cost) {
    const int ks = tile_ksplit<Cfg>(s, cus, part_cost);
    const long tiles = (long)ceil_div(s.M, Cfg::BM) * ceil_div(s.COg, Cfg::BN) * s.G * ks;
    const long per_cu = (tiles + cus - 1) / cus;
    const double lds = 1.0 + 0.5 * (double)(Cfg::TM + Cfg::TN) / (Cfg::TM * Cfg::TN);
    const double alone = Cfg::NT <= 256 && tiles <= cus ? 1.6 : 1.0;
    const double split = Cfg::NT > 256 && ks > 1 ? 1.01 + part_cost * ks : 1.0;  // as in tile_ksplit
    const double few_waves = Cfg::NT <= 256 ? 1.1 : 1.0;
    // measured: at equal padded area the half-height 1024-thread tile is 9 % slower than the full one
    const double half = std::is_same<Cfg, CfgWide4H>::value ? 1.08 : (std::is_same<Cfg, CfgOcc8>::value || std::is_same<Cfg, CfgOcc8W>::value ? 1e3 : 1.0);
    const double two_waves = op_heavy<Op>::value && std::is_same<Cfg, CfgMid>::value ? 1.08 : 1.0;
    return (double)per_cu * Cfg::BM * Cfg::BN * lds * alone * few_waves * half * two_waves * split / ks;
}

}  // namespace ndist

#include "fwd_skinny.h"

namespace ndist {

// Launches Op on the cheapest of the candidate tile configurations, or on the lanes-over-k kernel when the problem
// has too few outputs to fill the device with tiles.
template <bool CONV, class Op, class... Cfgs>
int launch_fwd_layouts(FwdParams P, hipStream_t st, int* chosen_kt = nullptr) {
    const Geom& s = P.s;
    static const char* force = getenv("NORM_DIST_TILE_CFG");
    if (force == nullptr && !P.implicit && skinny_applies(s)) return launch_skinny<Op>(P, st, chosen_kt);
    P.x_vec = (s.HW == 1 ? s.CIg % 4 == 0 : s.HW % 4 == 0) && ((uintptr_t)P.x % 16 == 0) &&
              (P.x2 == nullptr || (uintptr_t)P.x2 % 16 == 0);
    if (P.implicit) {
        P.x_vec = P.pm.OW % 4 == 0;  // scalar loads either way; this one says "four positions, one output row"
    }
    P.w_vec = s.CIg % 4 == 0 && ((uintptr_t)P.w % 16 == 0);
    P.y_vec = (s.HW == 1 ? s.COg % 4 == 0 : s.HW % 4 == 0) && ((uintptr_t)P.out % 16 == 0) &&
              (P.out2 == nullptr || (uintptr_t)P.out2 % 16 == 0) && (P.pos == nullptr || (uintptr_t)P.pos % 16 == 0) &&
              (P.pos2 == nullptr || (uintptr_t)P.pos2 % 16 == 0);
    const int cus = device_info().num_cu;
    const double part_cost = split_part_cost<Op>(s);
    const double costs[] = {tile_cost<Op, Cfgs>(s, cus, part_cost)...};
    int best = 0;
    for (int i = 1; i < (int)sizeof...(Cfgs); i++)
        if (costs[i] < costs[best]) best = i;
    // tuning aid: NORM_DIST_TILE_CFG=<index> forces the i-th candidate of the operator's list
    if (force != nullptr && force[0] >= '0' && force[0] - '0' < (int)sizeof...(Cfgs)) best = force[0] - '0';
    int idx = 0, rc = 2;
    ((idx++ == best ? (void)(P.kt = Cfgs::KT, rc = launch_cfg<Op, Cfgs, CONV>(P, tile_ksplit<Cfgs>(s, cus, part_cost), st)) : (void)0), ...);
    if (chosen_kt) *chosen_kt = P.kt;
    return rc;
}

template <class Op, class... Cfgs>
int launch_fwd(FwdParams P, hipStream_t st, int* chosen_kt = nullptr) {
    return launch_fwd_layouts<false, Op, Cfgs...>(P, st, chosen_kt);
}
// the same, with the implicit-patch kernels instantiated as well
template <class Op, class... Cfgs>
int launch_fwd_conv(FwdParams P, hipStream_t st) {
    return launch_fwd_layouts<true, Op, Cfgs...>(P, st, nullptr);
}

}  // namespace ndist
