// Forward of the infinity distance through "hot" k-tiles only (fully-connected layout, HW == 1).
// Serves inf_dist::forward / forward_nograd of the reference (core/cuda/inf_dist_cuda.cu:14-198,248-317) on data
// whose largest |x - w| are decided by few k: results are bit-identical to the dense kernels (values and codes).
//
// out[m, n] = max_k |x[m, k] - w[n, k]|.  With RX[m] = max_k |x[m, k]| and RW[n] = max_k |w[n, k]| (attained at kx,
// kw) the pair at kx shows out[m, n] >= RX[m] - RW[n], the pair at kw shows out[m, n] >= RW[n] - RX[m]; and inside a
// 32-wide k-tile t no pair exceeds bx[m, t] + bw[n, t], the largest magnitudes of the two rows inside the tile.  So a
// tile can hold the maximum of (m, n), or the first k that attains it, only if bx[m, t] + bw[n, t] reaches that lower
// bound.  Two separable sufficient tests follow, with MX = max_m RX[m], MW = max_n RW[n] (per group):
//   rows of x:  every tile with  bx[m, t] <  (RX[m] - MW) - MW  is dead for all n   (x decides: activations with few
//               outliers against small weights)
//   rows of w:  every tile with  bw[n, t] <  (RW[n] - MX) - MX  is dead for all m   (w decides: layers whose weights
//               carry a large planted entry per row)
// Either test alone is complete: under the first one no tile of w needs looking at beyond the tiles that are hot for
// the row of x, and vice versa.  A pre-pass (shared with the k-tile skipping kernels) gives RX, RW and the tile
// maxima; hot_plan_kernel turns them into one bit per (row, tile) for both tests, counts the bits and picks the
// cheaper test, or neither when too many tiles are hot (then the dense kernels run: everything downstream is queued
// gated on that decision, no host round trip).  inf_hot_kernel then walks, for every output, the hot tiles of its
// owner row in ascending k with the reference's own comparison (strict "greater": the lowest k wins ties, NaN never
// wins, 1e-10 floor with code 0), so values and codes need no second pass.
// Rounding: the thresholds are evaluated in double with a relative margin of 2^-22, which covers the fp32 rounding
// of the lower bound and of bx + bw (see hot_threshold).  A row that holds a NaN has a NaN row seed (the pair at its
// kx may not exist then): all its tiles are hot, and if it is a row of the other side nothing is dead at all.
#include <algorithm>
#include <atomic>
#include <stdlib.h>

#include "ndist_common.h"
#include "seed_outputs.h"

namespace ndist {

namespace {

// Threshold below which a tile maximum of the owner row makes the tile dead: own = R of the owner row, other = the
// largest R on the other side.  For a dead tile (b_own < A) and any row of the other side (b_other <= R_other <= other):
//   b_own + b_other < A + other = (own - other)(1 - 2^-22) <= (own - R_other)(1 - 2^-22),
// so fl32(b_own + b_other) <= (b_own + b_other)(1 + 2^-24) < (own - R_other)(1 - 2^-24) <= fl32(own - R_other) <= out:
// strictly below the output, hence neither its value nor the first k attaining it.  (Sums and differences of two
// floats are exact in the subnormal range, so the relative bounds hold there too.)  NaN (a row with a NaN, or
// inf - inf) and own < other give "nothing is dead".
__device__ __forceinline__ double hot_threshold(float own, float other) {
    const double a = ((double)own - (double)other) * (1.0 - 0x1p-22) - (double)other;
    return a == a ? a : -__builtin_inf();
}

// Largest row seed magnitude per group on both sides into LDS (sm[g] = MX, sm[G + g] = MW; infinite when a row of
// that side holds a NaN), computed by every workgroup for itself: the arrays are a few thousand floats.
__device__ __forceinline__ void hot_group_maxima(const float* __restrict__ seed_x, const float* __restrict__ seed_w,
                                                 const Geom& s, unsigned* sm) {
    for (int i = threadIdx.x; i < 2 * s.G; i += blockDim.x) sm[i] = 0u;
    __syncthreads();
    auto mag = [](float v) { v = fabsf(v); return v == v ? v : __builtin_inff(); };
    // magnitudes are non-negative floats: their bit patterns order like unsigned integers
    const long rows = (long)s.M * s.G, wrows = (long)s.COg * s.G;
    const int lane = threadIdx.x & 63;
    if (s.G == 1) {
        float mx = 0.f, mw = 0.f;
        for (long r = threadIdx.x; r < rows; r += blockDim.x) mx = fmaxf(mx, mag(seed_x[r]));
        for (long r = threadIdx.x; r < wrows; r += blockDim.x) mw = fmaxf(mw, mag(seed_w[r]));
#pragma unroll
        for (int d = 32; d >= 1; d >>= 1) {
            mx = fmaxf(mx, __shfl_xor(mx, d, 64));
            mw = fmaxf(mw, __shfl_xor(mw, d, 64));
        }
        if (lane == 0) {
            atomicMax(&sm[0], __float_as_uint(mx));
            atomicMax(&sm[1], __float_as_uint(mw));
        }
    } else {
        for (long r = threadIdx.x; r < rows; r += blockDim.x) atomicMax(&sm[r % s.G], __float_as_uint(mag(seed_x[r])));
        for (long r = threadIdx.x; r < wrows; r += blockDim.x)
            atomicMax(&sm[s.G + r / s.COg], __float_as_uint(mag(seed_w[r])));
    }
    __syncthreads();
}

// One kernel for the whole plan.  Every workgroup (1024 threads) first finds MX and MW of all groups, then its 16
// waves turn four rows each (rows of x first, then rows of w; their loads issued together) into hot-tile masks: bit
// t of a row's mask = tile t is hot (a row's record: one word naming its non-zero mask words, then the mask words).
// The workgroups leave their counts of hot (row, tile) entries per side in
// `partial`; the last one to finish (a ticket in dec[3], cleared by the row pre-pass) adds them up and decides:
//   dec[0] = 1: the rows of x select the tiles, 2: the rows of w, 0: too many hot tiles, the dense kernels run
//   (dec[4] / dec[5] then say which of them, see below).
// Cost of a side = its hot entries x the length of the other side.  mode: 1 always the cheaper side, 2 / 3 always
// the x / w side, else the cheaper side if it touches at most 1 / frac of all (row, column, tile) triples.
constexpr int kPlanRows = 32, kPlanRowsPerWave = kPlanRows / 16;
// What differs between two plans over the same weights (a layer's distance and its interval bounds in one call): the
// rows of the first operand with their statistics, and everything the plan writes.
struct PlanJob {
    const float* seed_x;
    const float* tile_x;
    uint32_t* mask_x;
    uint32_t* mask_w;
    int* dec;
    int* partial;
    const float* far_hi;  // interval bounds only
    const float* far_lo;
};
// Workgroups [0, nblk) serve job a, [nblk, 2 nblk) job b (launched with nblk workgroups when there is one job).
__global__ __launch_bounds__(1024) void hot_plan_kernel(const PlanJob ja, const PlanJob jb, int nblk,
                                                        const float* __restrict__ seed_w,
                                                        const float* __restrict__ tile_w, const Geom s, int ntile,
                                                        int nword, int mode, int frac, int dense_ok) {
    const bool second = (int)blockIdx.x >= nblk;
    const PlanJob& job = second ? jb : ja;
    const int bid = (int)blockIdx.x - (second ? nblk : 0);
    const float* __restrict__ seed_x = job.seed_x;
    const float* __restrict__ tile_x = job.tile_x;
    uint32_t* __restrict__ mask_x = job.mask_x;
    uint32_t* __restrict__ mask_w = job.mask_w;
    int* __restrict__ dec = job.dec;
    int* __restrict__ partial = job.partial;
    const float* __restrict__ far_hi = job.far_hi;
    const float* __restrict__ far_lo = job.far_lo;
    extern __shared__ unsigned sm[];  // 2 * G maxima
    __shared__ int cnt[2];
    __shared__ int is_last;
    __shared__ long long tot[2];
    if (threadIdx.x < 2) { cnt[threadIdx.x] = 0; tot[threadIdx.x] = 0; }
    const long rows = (long)s.M * s.G, wrows = (long)s.COg * s.G;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    constexpr int R = kPlanRowsPerWave;
    const float* tm[R];
    uint32_t* mk[R];
    double thr[R];
    bool valid[R], isw[R];
    long rr[R];
    int count[R];
    uint32_t nonzero[R];  // bit i: mask word i of the row has a hot tile (first word of the row's record)
    float own[R], fh[R], fl[R];
#pragma unroll
    for (int i = 0; i < R; i++) {
        const long r = (long)bid * kPlanRows + wave * R + i;
        valid[i] = r < rows + wrows;  // wave-uniform
        isw[i] = r >= rows;
        rr[i] = !valid[i] ? 0 : (isw[i] ? r - rows : r);
        tm[i] = (isw[i] ? tile_w : tile_x) + rr[i] * ntile;
        mk[i] = (isw[i] ? mask_w : mask_x) + rr[i] * (nword + 1);
        count[i] = 0;
        nonzero[i] = 0u;
        own[i] = fabsf(isw[i] ? seed_w[rr[i]] : seed_x[rr[i]]);
        fh[i] = fl[i] = 0.f;
        if (!isw[i] && far_hi != nullptr) {
            fh[i] = far_hi[rr[i]];
            fl[i] = far_lo[rr[i]];
        }
    }
    // The tile maxima of four steps (256 tiles of each row) are requested together, and the first such batch before
    // the group maxima are formed: the kernel is a chain of memory latencies, this leaves one for everything up to 8192 k.
    constexpr int STEPS = 4;
    float v[STEPS][R];
    auto fetch = [&](int t00) {
#pragma unroll
        for (int q = 0; q < STEPS; q++) {
            const int t = t00 + 64 * q + lane;
#pragma unroll
            for (int i = 0; i < R; i++) v[q][i] = valid[i] && t < ntile ? tm[i][t] : 0.f;
        }
    };
    fetch(0);
    hot_group_maxima(seed_x, seed_w, s, sm);
#pragma unroll
    for (int i = 0; i < R; i++) {
        const int g = isw[i] ? (int)(rr[i] / s.COg) : (int)(rr[i] % s.G);
        const float other = __uint_as_float(sm[isw[i] ? g : s.G + g]);
        thr[i] = hot_threshold(own[i], other);
        if (!isw[i] && far_hi != nullptr) {
            // interval bounds, rows of the box: the two reductions have their own lower bounds, far_hi - RW for the
            // upper one and far_lo - RW for the lower one; a tile is dead when it is dead for both
            const double tu = hot_threshold(fh[i], other), tl = hot_threshold(fl[i], other);
            thr[i] = own[i] == own[i] ? (tu < tl ? tu : tl) : -__builtin_inf();
        }
    }
    for (int t00 = 0; t00 < nword * 32; t00 += 64 * STEPS) {
        if (t00 > 0) fetch(t00);
#pragma unroll
        for (int q = 0; q < STEPS; q++) {
            const int t0 = t00 + 64 * q, t = t0 + lane;
            if (t0 >= nword * 32) break;  // the same for all lanes
#pragma unroll
            for (int i = 0; i < R; i++) {
                const bool hot = valid[i] && t < ntile && !((double)v[q][i] < thr[i]);
                const unsigned long long bits = __builtin_amdgcn_ballot_w64(hot);
                count[i] += __popcll(bits);
                const int wi = t0 >> 5;
                nonzero[i] |= ((uint32_t)bits != 0u ? 1u << (wi & 31) : 0u) | ((bits >> 32) != 0ull ? 1u << ((wi + 1) & 31) : 0u);
                if (lane == 0 && valid[i]) {
                    mk[i][1 + wi] = (uint32_t)bits;
                    if (wi + 1 < nword) mk[i][2 + wi] = (uint32_t)(bits >> 32);
                }
            }
        }
    }
    if (lane == 0) {
#pragma unroll
        for (int i = 0; i < R; i++) {
            if (!valid[i]) continue;
            mk[i][0] = nonzero[i];
            if (count[i] != 0) atomicAdd(&cnt[isw[i] ? 1 : 0], count[i]);
        }
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        partial[2 * bid] = cnt[0];
        partial[2 * bid + 1] = cnt[1];
        __threadfence();  // the counts are visible device-wide before the ticket is taken
        is_last = atomicAdd(&dec[3], 1) == nblk - 1;
    }
    __syncthreads();
    if (!is_last || wave != 0) return;
    // the last workgroup's first wave adds the counts up (butterfly over the lanes) and decides
    __threadfence();
    long long cx = 0, cw = 0;
    for (int b = lane; b < nblk; b += 64) {
        cx += __atomic_load_n(&partial[2 * b], __ATOMIC_RELAXED);
        cw += __atomic_load_n(&partial[2 * b + 1], __ATOMIC_RELAXED);
    }
#pragma unroll
    for (int d = 32; d >= 1; d >>= 1) {
        cx += __shfl_xor(cx, d, 64);
        cw += __shfl_xor(cw, d, 64);
    }
    if (lane == 0) {
        tot[0] = cx;
        tot[1] = cw;
        const long long costx = tot[0] * s.COg, costw = tot[1] * s.M;
        const long long total = (long long)s.M * s.G * s.COg * ntile;
        int choice = costx <= costw ? 1 : 2;
        if (mode == 2) choice = 1;
        else if (mode == 3) choice = 2;
        else if (mode != 1 && (costx <= costw ? costx : costw) * frac > total) choice = 0;
        dec[0] = choice;
        // Which of the two dense kernels runs when the hot tiles do not: with (nearly) every tile hot on both sides
        // under the separable test, the kernel that checks tile bounds has nothing to drop and only pays for its
        // bounds, votes and flags (a third per stage): the plain tiled kernel takes over.  Gate words, 0 = run.
        const bool dense = dense_ok != 0 && tot[0] * 10 > (long long)s.M * s.G * ntile * 9 &&
                           tot[1] * 10 > (long long)s.COg * s.G * ntile * 9;
        dec[4] = choice != 0 || dense ? 1 : 0;   // tile-skipping kernel (and the output seeds it starts from)
        dec[5] = choice != 0 || !dense ? 1 : 0;  // plain kernel
        dec[1] = (int)(tot[0] > 0x7fffffff ? 0x7fffffff : tot[0]);  // for inspection
        dec[2] = (int)(tot[1] > 0x7fffffff ? 0x7fffffff : tot[1]);
    }
}

// Value of the partner lane in a merge of the eight lanes that share a row: step 1 and 2 are the butterfly inside a
// quad (quad_perm), step 4 pairs lane i of one quad with lane 7 - i of the other (row_half_mirror) -- by then all four
// lanes of a quad hold the same state, so any lane of the other quad will do.  DPP moves: no LDS round trip.
template <typename T>
__device__ __forceinline__ T partner8(T v, int d) {
    static_assert(sizeof(T) == 4, "32-bit values");
    const int i = __builtin_bit_cast(int, v);
    int r;
    if (d == 1) r = __builtin_amdgcn_update_dpp(0, i, 0xB1, 0xf, 0xf, true);        // quad_perm [1, 0, 3, 2]
    else if (d == 2) r = __builtin_amdgcn_update_dpp(0, i, 0x4E, 0xf, 0xf, true);   // quad_perm [2, 3, 0, 1]
    else r = __builtin_amdgcn_update_dpp(0, i, 0x141, 0xf, 0xf, true);              // row_half_mirror
    return __builtin_bit_cast(T, r);
}

// The two operators as policies of the walk: per-output state, one pair, the merge of two lanes' states (the larger
// value, among equal values the lower k; "nothing found" carries the operator's initial code, which no found pair
// can tie with because a pair must beat the floor strictly), the outputs.
// For the merges a code travels as a rank: higher for lower k, sign flag in the lowest bit.  (value, rank) pairs of
// positive values then order as 64-bit integers -- larger value first, among equal values the lower k -- and a merge
// step is one 64-bit compare and two selects per reduction.
__device__ __forceinline__ uint32_t code_to_rank(uint32_t code) { return ((0x7fffffffu - (code & ~kSignBit)) << 1) | (code >> 31); }
__device__ __forceinline__ uint32_t rank_to_code(uint32_t rank) { return (0x7fffffffu - (rank >> 1)) | (rank << 31); }
__device__ __forceinline__ bool pair_beats(float ov, uint32_t orank, float v, uint32_t rank) {
    const unsigned long long a = ((unsigned long long)__float_as_uint(ov) << 32) | orank;
    const unsigned long long b = ((unsigned long long)__float_as_uint(v) << 32) | rank;
    return a > b;
}

template <bool TRACK>
struct HotInf {
    static constexpr int kSeedLds = kSeedTileFloats;
    __device__ static __forceinline__ void seed_outputs(const float* x, long, const float* w, const Geom& s,
                                                        const OutputSeedJob& job, unsigned id, float* lds) {
        norm_seed_outputs_block(x, w, s, job, id, lds);
    }
    static constexpr int kMinWaves = TRACK ? 5 : 7;  // per SIMD: what the kernel reaches by itself  // out = max(1e-10, max_k |x - w|), code = k | sign flag (core/cuda/inf_dist_cuda.cu:131-132,173-177)
    static constexpr int NX = 1, NF = 1, NI = TRACK ? 1 : 0;
    struct State { float best; uint32_t code; };
    __device__ static __forceinline__ void init(State& a) { a.best = kEps; a.code = 0; }
    __device__ static __forceinline__ void pair(State& a, float xv, float, float wv, int k) {
        const float d = xv - wv, v = fabsf(d);
        if constexpr (TRACK) {
            if (v > a.best) { a.best = v; a.code = (uint32_t)k | (d >= 0 ? 0u : kSignBit); }
        } else {
            a.best = fmaxf(a.best, v);
        }
    }
    // around the merge steps of a state: its code as a rank and back
    __device__ static __forceinline__ void pre_merge(State& a) {
        if constexpr (TRACK) a.code = code_to_rank(a.code);
    }
    __device__ static __forceinline__ void post_merge(State& a) {
        if constexpr (TRACK) a.code = rank_to_code(a.code);
    }
    __device__ static __forceinline__ void merge_xor(State& a, int d) {
        const float ob = partner8(a.best, d);
        if constexpr (TRACK) {
            const uint32_t oc = partner8(a.code, d);
            const bool take = pair_beats(ob, oc, a.best, a.code);
            a.best = take ? ob : a.best;
            a.code = take ? oc : a.code;
        } else {
            a.best = fmaxf(a.best, ob);
        }
    }
    __device__ static __forceinline__ void select(State& a, const State& b, bool c) {
        a.best = c ? b.best : a.best;
        a.code = c ? b.code : a.code;
    }
    __device__ static __forceinline__ void outputs(const State& a, float* f, uint32_t* i) {
        f[0] = a.best;
        if constexpr (TRACK) i[0] = a.code;
    }
};

template <bool TRACK>
struct HotBound {
    static constexpr int kSeedLds = 2 * kSeedTileFloats;
    __device__ static __forceinline__ void seed_outputs(const float* x, long x2off, const float* w, const Geom& s,
                                                        const OutputSeedJob& job, unsigned id, float* lds) {
        bound_seed_outputs_block(x, x + x2off, w, s, job, id, lds);
    }
    // per SIMD: with the codes the kernel would take 136 registers and run 3; held to 128 (a few cold values spill) it
    // is 12 % faster
    static constexpr int kMinWaves = 4;  // interval bounds (core/cuda/bound_inf_dist_cuda.cu:63,148-151,203-213,225-232)
    static constexpr int NX = 2, NF = 2, NI = TRACK ? 2 : 0;
    struct State { float lo, hi; uint32_t wl, wu; };
    __device__ static __forceinline__ void init(State& a) { a.lo = -kEps; a.hi = kEps; a.wl = kNoGradId; a.wu = 0; }
    __device__ static __forceinline__ void pair(State& a, float xl, float xu, float wv, int k) {
        if (xl > xu) xl = xu = (xl + xu) * 0.5f;  // an inverted box collapses to its midpoint
        const float t1 = wv - xl, t2 = xu - wv;
        const float mn = fminf(t1, t2), mx = fmaxf(t1, t2);
        if constexpr (TRACK) {
            const uint32_t code = (uint32_t)k | (t1 <= t2 ? 0u : kSignBit);
            if (mn < a.lo) { a.lo = mn; a.wl = code; }
            if (mx > a.hi) { a.hi = mx; a.wu = code; }
        } else {
            a.lo = fminf(a.lo, mn);
            a.hi = fmaxf(a.hi, mx);
        }
    }
    // around the merge steps of a state: the lower reduction negated (a maximum of positive values like the upper
    // one), the codes as ranks
    __device__ static __forceinline__ void pre_merge(State& a) {
        if constexpr (TRACK) {
            a.lo = -a.lo;
            a.wl = code_to_rank(a.wl);
            a.wu = code_to_rank(a.wu);
        }
    }
    __device__ static __forceinline__ void post_merge(State& a) {
        if constexpr (TRACK) {
            a.lo = -a.lo;
            a.wl = rank_to_code(a.wl);
            a.wu = rank_to_code(a.wu);
        }
    }
    __device__ static __forceinline__ void merge_xor(State& a, int d) {
        const float ol = partner8(a.lo, d), oh = partner8(a.hi, d);
        if constexpr (TRACK) {
            const uint32_t cl = partner8(a.wl, d), cu = partner8(a.wu, d);
            const bool tl = pair_beats(ol, cl, a.lo, a.wl);
            const bool tu = pair_beats(oh, cu, a.hi, a.wu);
            a.lo = tl ? ol : a.lo;
            a.wl = tl ? cl : a.wl;
            a.hi = tu ? oh : a.hi;
            a.wu = tu ? cu : a.wu;
        } else {
            a.lo = fminf(a.lo, ol);
            a.hi = fmaxf(a.hi, oh);
        }
    }
    __device__ static __forceinline__ void select(State& a, const State& b, bool c) {
        a.lo = c ? b.lo : a.lo;
        a.hi = c ? b.hi : a.hi;
        a.wl = c ? b.wl : a.wl;
        a.wu = c ? b.wu : a.wu;
    }
    __device__ static __forceinline__ void outputs(const State& a, float* f, uint32_t* i) {
        f[0] = -a.lo;
        f[1] = a.hi;
        if constexpr (TRACK) { i[0] = a.wl; i[1] = a.wu; }
    }
};

// One wave: the hot tiles of one owner row (bits of mk, ascending k) against 64 rows of the other side.  Eight lanes
// share a row of the other side and split a 32-wide tile into 16-byte pieces (a load instruction then covers eight
// whole 128-byte rows instead of 64 different cache lines), lane group q of the wave serves the rows q, q + 8, ...,
// q + 8 * (kHotSlots - 1) past `oth`, `stride` floats apart (`nrow` of them exist; the others re-read the first row and are
// discarded by the caller).  X_OWNS: the owner is the row of x.  x has a second array at distance `x2off` floats
// for the interval bounds (P::NX == 2).  Every lane ends with the result of row 8 * (lane & 7) + (lane >> 3).
constexpr int kHotSlots = 4;               // rows of the other side per lane group
constexpr int kHotRows = 8 * kHotSlots;    // rows of the other side per wave
template <class P, bool X_OWNS>
__device__ __forceinline__ void hot_walk(const float* __restrict__ own, const float* __restrict__ oth, long x2off,
                                         long stride, int nrow, const uint32_t* __restrict__ mk, int nword, int K,
                                         bool vec, typename P::State& res, bool ahead = false, uint32_t summary = 0,
                                         uint32_t first_word = 0) {
    using State = typename P::State;
    constexpr bool TWO = P::NX == 2;
    const int lane = threadIdx.x & 63, sub = lane & 7, q = lane >> 3;
    State st[kHotSlots];
    const float* rowp[kHotSlots];
#pragma unroll
    for (int j = 0; j < kHotSlots; j++) {
        P::init(st[j]);
        const int row = q + 8 * j;
        rowp[j] = oth + (long)(row < nrow ? row : 0) * stride;
    }
    // mk[0] names the mask words that hold a hot tile (when there are at most 32 of them): usually a single one, so
    // the walk costs two dependent loads instead of one per word
    // (`ahead`: the caller has fetched the summary and the first word it names already, for several rows at once)
    uint32_t pending = ahead ? summary : mk[0];
    int wi = -1;
    bool first = ahead;
    while (true) {
        if (nword <= 32) {
            if (pending == 0) break;
            wi = __builtin_ctz(pending);
            pending &= pending - 1;
        } else if (++wi >= nword) {
            break;
        }
        uint32_t bits = first ? first_word : mk[1 + wi];
        first = false;
        while (bits != 0) {
            const int k0 = (wi * 32 + __builtin_ctz(bits)) * 32 + 4 * sub;
            bits &= bits - 1;
            if (vec && k0 + 4 <= K) {
                const float4 o = *reinterpret_cast<const float4*>(own + k0);
                float4 o2 = o;
                if constexpr (TWO && X_OWNS) o2 = *reinterpret_cast<const float4*>(own + x2off + k0);
                float4 v[kHotSlots], v2[TWO && !X_OWNS ? kHotSlots : 1];
#pragma unroll
                for (int j = 0; j < kHotSlots; j++) {
                    v[j] = *reinterpret_cast<const float4*>(rowp[j] + k0);
                    if constexpr (TWO && !X_OWNS) v2[j] = *reinterpret_cast<const float4*>(rowp[j] + x2off + k0);
                }
#pragma unroll
                for (int j = 0; j < kHotSlots; j++) {
                    if constexpr (X_OWNS) {
                        P::pair(st[j], o.x, o2.x, v[j].x, k0 + 0);
                        P::pair(st[j], o.y, o2.y, v[j].y, k0 + 1);
                        P::pair(st[j], o.z, o2.z, v[j].z, k0 + 2);
                        P::pair(st[j], o.w, o2.w, v[j].w, k0 + 3);
                    } else {
                        const float4 u = TWO ? v2[TWO && !X_OWNS ? j : 0] : v[j];
                        P::pair(st[j], v[j].x, u.x, o.x, k0 + 0);
                        P::pair(st[j], v[j].y, u.y, o.y, k0 + 1);
                        P::pair(st[j], v[j].z, u.z, o.z, k0 + 2);
                        P::pair(st[j], v[j].w, u.w, o.w, k0 + 3);
                    }
                }
            } else {
                const int k1 = min(k0 + 4, K);
                for (int k = k0; k < k1; k++) {
                    const float o = own[k], o2 = TWO && X_OWNS ? own[x2off + k] : o;
#pragma unroll
                    for (int j = 0; j < kHotSlots; j++) {
                        if constexpr (X_OWNS) P::pair(st[j], o, o2, rowp[j][k], k);
                        else P::pair(st[j], rowp[j][k], TWO ? rowp[j][x2off + k] : 0.f, o, k);
                    }
                }
            }
        }
    }
    // the eight lanes of a row merge
#pragma unroll
    for (int j = 0; j < kHotSlots; j++) {
        P::pre_merge(st[j]);
#pragma unroll
        for (int d = 1; d < 8; d <<= 1) P::merge_xor(st[j], d);
        P::post_merge(st[j]);
    }
    res = st[0];
#pragma unroll
    for (int j = 1; j < kHotSlots; j++) P::select(res, st[j], sub == j);
}

struct HotOut {
    float* f[2];
    int32_t* i[2];
};

// The kernel that computes the outputs from the hot tiles, for whichever side the plan chose.
//   dec[0] == 1, the rows of x own: a workgroup takes one row of x and 256 columns (64 per wave).
//   dec[0] == 2, the rows of w own: a workgroup takes 16 rows of w (four per wave, one after the other) and 64 rows
//   of x; the results turn around in LDS so that every row of the output is written 16 columns at a time.
//   dec[0] == 0, the dense kernels queued behind this one run: the first seed_blocks workgroups compute the output
//   seeds those kernels start from (a launch of its own otherwise; on the hot path every launch that finds itself
//   gated off costs about as much as the plan kernel's decision saves).
// x2off: distance in floats from x (the lower input bound) to the upper one (interval bounds only).
template <class P>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(P::kMinWaves))) void hot_kernel(const float* __restrict__ x, long x2off, const float* __restrict__ w,
                                                  const Geom s, const uint32_t* __restrict__ mask_x,
                                                  const uint32_t* __restrict__ mask_w, int nword, int vec, const HotOut out,
                                                  const int* __restrict__ dec, unsigned grid_rows, unsigned grid_cols,
                                                  const OutputSeedJob seeds, unsigned seed_blocks) {
    constexpr int NF = P::NF, NI = P::NI;
    // one array for both roles: [NF][kHotRows][17] values and [NI][kHotRows][17] codes, or the tiles of the seeds
    constexpr int kTurn = (NF + NI) * kHotRows * 17;
    __shared__ float lds[kTurn > P::kSeedLds ? kTurn : P::kSeedLds];
    float (*tv)[kHotRows][17] = reinterpret_cast<float (*)[kHotRows][17]>(lds);
    uint32_t (*tc)[kHotRows][17] = reinterpret_cast<uint32_t (*)[kHotRows][17]>(lds + NF * kHotRows * 17);
    const int choice = dec[0];
    if (choice == 0) {
        if (dec[4] == 0 && blockIdx.x < seed_blocks) P::seed_outputs(x, x2off, w, s, seeds, blockIdx.x, lds);
        return;
    }
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    // the row of the other side whose result this lane ends up with (lanes with (lane & 7) >= kHotSlots: none)
    const int mine = 8 * (lane & 7) + (lane >> 3);
    const bool reports = (lane & 7) < kHotSlots;
    typename P::State res;
    float fv[NF];
    uint32_t iv[NI > 0 ? NI : 1];
    if (choice == 1) {
        if (blockIdx.x >= grid_rows) return;
        const int nchunk = ceil_div(s.COg, 4 * kHotRows);
        const long r = blockIdx.x / (unsigned)nchunk;  // row (m, g) of x
        const int n0 = (int)(blockIdx.x % (unsigned)nchunk) * 4 * kHotRows + wave * kHotRows;
        if (n0 >= s.COg) return;  // whole waves
        const int g = (int)(r % s.G);
        hot_walk<P, true>(x + r * s.CIg, w + ((long)g * s.COg + n0) * s.CIg, x2off, s.CIg, min(kHotRows, s.COg - n0),
                          mask_x + r * (nword + 1), nword, s.CIg, vec != 0, res);
        const int n = n0 + mine;
        if (reports && n < s.COg) {
            P::outputs(res, fv, iv);
#pragma unroll
            for (int c = 0; c < NF; c++) out.f[c][r * s.COg + n] = fv[c];
#pragma unroll
            for (int c = 0; c < NI; c++) out.i[c][r * s.COg + n] = (int32_t)iv[c];
        }
    } else if (choice == 2) {
        if (blockIdx.x >= grid_cols) return;
        const int nmb = ceil_div(s.M, kHotRows), nnb = ceil_div(s.COg, 16);
        unsigned id = blockIdx.x;
        const int mb = (int)(id % (unsigned)nmb);
        id /= (unsigned)nmb;
        const int nb = (int)(id % (unsigned)nnb), g = (int)(id / (unsigned)nnb);
        const int m0 = mb * kHotRows;
        // HW == 1: row m of group g of x starts at (m * G + g) * CIg, consecutive rows are G * CIg apart
        // The four rows of a wave are walked one after the other, each a chain of dependent loads (summary, mask
        // word, tile pieces): the summaries of all four, then the first words they name, are fetched up front.
        const bool ahead = nword <= 32;
        uint32_t summary[4] = {0u, 0u, 0u, 0u}, word0[4] = {0u, 0u, 0u, 0u};
        if (ahead) {
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const int n = min(nb * 16 + wave * 4 + i, s.COg - 1);
                summary[i] = mask_w[((long)g * s.COg + n) * (nword + 1)];
            }
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const int n = min(nb * 16 + wave * 4 + i, s.COg - 1);
                const int w0 = summary[i] != 0u ? __builtin_ctz(summary[i]) : 0;
                word0[i] = mask_w[((long)g * s.COg + n) * (nword + 1) + 1 + w0];
            }
        }
        for (int i = 0; i < 4; i++) {
            const int c = wave * 4 + i, n = nb * 16 + c;
            P::init(res);
            if (n < s.COg) {  // wave-uniform
                const long wrow = (long)g * s.COg + n;
                hot_walk<P, false>(w + wrow * s.CIg, x + ((long)m0 * s.G + g) * s.CIg, x2off, (long)s.CIg * s.G,
                                   min(kHotRows, s.M - m0), mask_w + wrow * (nword + 1), nword, s.CIg, vec != 0, res,
                                   ahead, summary[i], word0[i]);
            }
            P::outputs(res, fv, iv);
            if (reports) {
#pragma unroll
                for (int e = 0; e < NF; e++) tv[e][mine][c] = fv[e];
#pragma unroll
                for (int e = 0; e < NI; e++) tc[e][mine][c] = iv[e];
            }
        }
        __syncthreads();
        const int mr = threadIdx.x >> 2, mo = m0 + mr, c0 = (threadIdx.x & 3) * 4;
        if (mr < kHotRows && mo < s.M) {
#pragma unroll
            for (int j = 0; j < 4; j++) {
                const int n = nb * 16 + c0 + j;
                if (n < s.COg) {
                    const long o = ((long)mo * s.G + g) * s.COg + n;
#pragma unroll
                    for (int e = 0; e < NF; e++) out.f[e][o] = tv[e][mr][c0 + j];
#pragma unroll
                    for (int e = 0; e < NI; e++) out.i[e][o] = (int32_t)tc[e][mr][c0 + j];
                }
            }
        }
    }
}

int env_hot_mode() {
    const char* v = getenv("NORM_DIST_HOT");
    return v == nullptr || v[0] < '0' || v[0] > '3' ? -1 : v[0] - '0';
}
const int g_env_hot = env_hot_mode();
thread_local int t_hot_mode = g_env_hot;  // per calling host thread, like the other overrides

}  // namespace

void set_hot_mode(int mode) { t_hot_mode = mode < 0 || mode > 3 ? g_env_hot : mode; }
int hot_mode() { return t_hot_mode; }

static int plan_blocks(const Geom& s) {
    return (int)(((long)s.M * s.G + (long)s.COg * s.G + kPlanRows - 1) / kPlanRows);
}

bool hot_forward_applies(const Geom& s) { return hot_mode() != 0 && s.HW == 1 && s.G <= 4096; }

size_t hot_scratch_floats(const Geom& s) {
    const size_t nword = (size_t)ceil_div(ceil_div(s.CIg, 32), 32);
    return 8 + 2 * (size_t)plan_blocks(s) + (nword + 1) * ((size_t)s.M * s.G + (size_t)s.COg * s.G);
}

// Where the plan's results lie in an operator's hot scratch (`base`).
struct HotLayout {
    int* dec;  // [0] decision, [1], [2] hot entries per side, [3] ticket (cleared by the row pre-pass), [4], [5] gate
               // words of the two dense kernels (0 = run)
    int* partial;
    uint32_t* mask_x;
    uint32_t* mask_w;
    int nword, nblk;
};
static HotLayout hot_layout(const Geom& s, const SeedBuffers& sb, float* base) {
    HotLayout h{};
    h.nword = ceil_div(sb.ntile, 32);
    h.nblk = plan_blocks(s);
    h.dec = reinterpret_cast<int*>(base);
    h.partial = h.dec + 8;
    h.mask_x = reinterpret_cast<uint32_t*>(h.partial + 2 * h.nblk);
    h.mask_w = h.mask_x + (long)s.M * s.G * (h.nword + 1);
    return h;
}
static PlanJob plan_job(const HotLayout& h, const SeedBuffers& sb, bool box) {
    return PlanJob{sb.seed_x, sb.tile_x, h.mask_x, h.mask_w, h.dec, h.partial, box ? sb.far_hi : nullptr,
                   box ? sb.far_lo : nullptr};
}
// at most 1 / 12 of all (row, column, tile) triples: measured at 5120 x 5120 with 512 and with 64 rows, the dense
// kernels are the faster ones from about a tenth on
constexpr int kHotFraction = 12;

int launch_joint_hot_plan(const Geom& s, const SeedBuffers& sb, float* base, const SeedBuffers& sb_box, float* base_box,
                          hipStream_t st) {
    const HotLayout ha = hot_layout(s, sb, base), hb = hot_layout(s, sb_box, base_box);
    hipLaunchKernelGGL(hot_plan_kernel, dim3(2 * ha.nblk), dim3(1024), 2 * s.G * sizeof(unsigned), st,
                       plan_job(ha, sb, false), plan_job(hb, sb_box, true), ha.nblk, sb.seed_w, sb.tile_w, s, sb.ntile,
                       ha.nword, hot_mode(), kHotFraction, skip_forced_on() ? 0 : 1);
    return hip_failed(hipGetLastError()) ? 4 : 0;
}

static int launch_hot(const float* x, const float* x2, const float* w, const Geom& s, const SeedBuffers& sb, float* base,
                      const HotOut& out, bool track, hipStream_t st, const int** decision, bool with_seeds,
                      bool plan_done) {
    const HotLayout h = hot_layout(s, sb, base);
    const int nword = h.nword;
    const long rows = (long)s.M * s.G;
    int* dec = h.dec;
    uint32_t* mask_x = h.mask_x;
    uint32_t* mask_w = h.mask_w;
    *decision = dec;
    if (!plan_done) {
        const PlanJob job = plan_job(h, sb, x2 != nullptr);
        hipLaunchKernelGGL(hot_plan_kernel, dim3(h.nblk), dim3(1024), 2 * s.G * sizeof(unsigned), st, job, job, h.nblk,
                           sb.seed_w, sb.tile_w, s, sb.ntile, nword, hot_mode(), kHotFraction, skip_forced_on() ? 0 : 1);
    }
    int vec = s.CIg % 4 == 0 && (uintptr_t)x % 16 == 0 && (uintptr_t)w % 16 == 0;
    if (x2 != nullptr) vec = vec && (uintptr_t)x2 % 16 == 0;
    const long x2off = x2 != nullptr ? (long)(((intptr_t)x2 - (intptr_t)x) / (intptr_t)sizeof(float)) : 0;
    const unsigned grid_r = (unsigned)(rows * ceil_div(s.COg, 4 * kHotRows));
    const unsigned grid_c = (unsigned)((long)ceil_div(s.M, kHotRows) * ceil_div(s.COg, 16) * s.G);
    const OutputSeedJob job = output_seed_job(s, sb);
    const unsigned seed_blocks = with_seeds ? (unsigned)((long)job.nmb * job.nnb * s.G) : 0u;
    const dim3 grid(std::max(std::max(grid_r, grid_c), seed_blocks));
#define NDIST_HOT(POLICY) \
    hipLaunchKernelGGL(hot_kernel<POLICY>, grid, dim3(256), 0, st, x, x2off, w, s, mask_x, mask_w, nword, vec, out, dec, \
                       grid_r, grid_c, job, seed_blocks)
    if (x2 == nullptr) {
        if (track) NDIST_HOT(HotInf<true>);
        else NDIST_HOT(HotInf<false>);
    } else {
        if (track) NDIST_HOT(HotBound<true>);
        else NDIST_HOT(HotBound<false>);
    }
#undef NDIST_HOT
    return hip_failed(hipGetLastError()) ? 4 : 0;
}

int launch_inf_hot(const float* x, const float* w, const Geom& s, const SeedBuffers& sb, float* base, float* out,
                   int32_t* pos, hipStream_t st, const int** decision, bool with_seeds, bool plan_done) {
    const HotOut o{{out, nullptr}, {pos, nullptr}};
    return launch_hot(x, nullptr, w, s, sb, base, o, pos != nullptr, st, decision, with_seeds, plan_done);
}

int launch_bound_hot(const float* xl, const float* xu, const float* w, const Geom& s, const SeedBuffers& sb, float* base,
                     float* yl, float* yu, int32_t* pl, int32_t* pu, hipStream_t st, const int** decision,
                     bool with_seeds, bool plan_done) {
    const HotOut o{{yl, yu}, {pl, pu}};
    return launch_hot(xl, xu, w, s, sb, base, o, pl != nullptr, st, decision, with_seeds, plan_done);
}

}  // namespace ndist
