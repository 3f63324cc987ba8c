// Fused finite-p backward: exponent p-1 = 7 and the general (non-integral or large) exponent, the pre-pass and the
// host-side driver.
#include <cstdlib>

#include "bwd_norm.h"

namespace ndist {

template <> int launch_bwd_ip<7>(const BwdPtrs& a, const BwdParams& P, int cfg, int grid, hipStream_t st) { return launch_bwd_ip_impl<7>(a, P, cfg, grid, st); }
template <> int launch_bwd_ip<-1>(const BwdPtrs& a, const BwdParams& P, int cfg, int grid, hipStream_t st) { return launch_bwd_ip_impl<-1>(a, P, cfg, grid, st); }
template <> int launch_bwd_ip<-3>(const BwdPtrs& a, const BwdParams& P, int cfg, int grid, hipStream_t st) { return launch_bwd_ip_impl<-3>(a, P, cfg, grid, st); }
template <> int launch_bwd_ip<-2>(const BwdPtrs& a, const BwdParams& P, int cfg, int grid, hipStream_t st) { return launch_bwd_ip_impl<-2>(a, P, cfg, grid, st); }
template <> int launch_bwd_ip<-5>(const BwdPtrs& a, const BwdParams& P, int cfg, int grid, hipStream_t st) { return launch_bwd_ip_impl<-5>(a, P, cfg, grid, st); }
// skipping by bounds (row-split configurations only)
template <> int launch_bwd_ip<-4>(const BwdPtrs& a, const BwdParams& P, int cfg, int grid, hipStream_t st) {
    if (cfg > 2) return 2;  // not instantiated for the small-batch kernel
    if (cfg == 2) {  // 256 bytes more LDS than the other variants: three 4-wave workgroups per compute unit, not four
        const int fit = 3 * device_info().num_cu;
        grid = grid < fit ? grid : fit;
    }
#define NDIST_BWD_BOUNDS(WITH_W, C)                                                                                  \
    hipLaunchKernelGGL((bwd_fused_kernel<-4, WITH_W, kBwdCfgRows[C], kBwdCfgWaves[C]>), dim3(grid),                  \
                       dim3(64 * kBwdCfgWaves[C]), 0, st, a.x, a.w, a.aT, a.gx, a.gw, P)
    KernelTimer timer(st);
    if (a.gw != nullptr) {
        if (cfg == 0) NDIST_BWD_BOUNDS(true, 0);
        else if (cfg == 1) NDIST_BWD_BOUNDS(true, 1);
        else NDIST_BWD_BOUNDS(true, 2);
    } else {
        if (cfg == 0) NDIST_BWD_BOUNDS(false, 0);
        else if (cfg == 1) NDIST_BWD_BOUNDS(false, 1);
        else NDIST_BWD_BOUNDS(false, 2);
    }
#undef NDIST_BWD_BOUNDS
    return hip_failed(hipGetLastError()) ? 4 : 0;
}

// Second step of the reproducible grad_input, over the (group, slab, row chunk) blocks.  The persistent
// workgroups of the main kernel took the unit ranges [g * total / nwg, (g + 1) * total / nwg); a block whose units lie
// in one range was stored by that workgroup, every other block is the sum, in workgroup order, of the shares its
// workgroups left in `part`.
__global__ __launch_bounds__(256) void bwd_gx_fixup_kernel(const float* __restrict__ part, float* __restrict__ GX,
                                                           const BwdParams P, int nwg, int rows_per_wg) {
    const Geom& s = P.s;
    // (1024 elements of a block per workgroup)
    const int nchunk = (rows_per_wg * kBwdSlab + 1023) / 1024;
    const int e0 = (int)(blockIdx.x % (unsigned)nchunk) * 1024;
    auto begin = [&](long g) { return g * P.total / nwg; };
    auto owner = [&](long u) {  // the workgroup whose range holds unit u
        long g = u * nwg / P.total;
        g = g < 0 ? 0 : (g > nwg - 1 ? nwg - 1 : g);
        while (g > 0 && begin(g) > u) g--;
        while (g + 1 < nwg && begin(g + 1) <= u) g++;
        return g;
    };
    // The grid runs over the boundaries between workgroups, not over all blocks: only a block with a boundary inside
    // is split (with few output columns the blocks are short and almost all of them whole).  A block that holds
    // several boundaries belongs to the first of them.
    const long first = blockIdx.x / (unsigned)nchunk;  // the boundary between workgroups `first` and `first` + 1
    const long ub = begin(first + 1);
    if (ub % P.ncc == 0) return;                       // it falls between two blocks
    const long sr = ub / P.ncc, b0 = sr * P.ncc, b1 = b0 + P.ncc;
    const long g_lo = owner(b0), g_hi = owner(b1 - 1);
    if (g_lo != first || g_lo == g_hi) return;
    const int rc = (int)(sr % P.nrc);
    const int gs = (int)(sr / P.nrc);
    const int grp = gs / P.nslab, ci0 = (gs - grp * P.nslab) * kBwdSlab;
    if (s.HW == 1 && s.CIg % 4 == 0 && (reinterpret_cast<uintptr_t>(GX) & 15) == 0) {
        // four consecutive ci per thread: 16-byte loads of every share, all of them on their way before the first add
        const int e = e0 + 4 * threadIdx.x;
        if (e >= rows_per_wg * kBwdSlab) return;
        const int r = e / kBwdSlab, l = e - r * kBwdSlab;
        const int m = rc * rows_per_wg + r, ci = ci0 + l;
        if (m >= s.M || ci >= s.CIg) return;
        float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
        for (long g = g_lo; g <= g_hi; g++) {
            const int slot = sr == begin(g) / P.ncc ? 0 : 1;
            const float4 t = *reinterpret_cast<const float4*>(part + ((g * 2 + slot) * rows_per_wg + r) * kBwdSlab + l);
            v = make_float4(v.x + t.x, v.y + t.y, v.z + t.z, v.w + t.w);
        }
        *reinterpret_cast<float4*>(GX + x_off(s, m, grp, ci, 0)) = v;
        return;
    }
    for (int e = e0 + threadIdx.x; e < min(e0 + 1024, rows_per_wg * kBwdSlab); e += 256) {
        const int r = e / kBwdSlab, l = e - r * kBwdSlab;
        const int m = rc * rows_per_wg + r, ci = ci0 + l;
        if (m >= s.M || ci >= s.CIg) continue;
        float v = 0.f;
        for (long g = g_lo; g <= g_hi; g++) {
            const int slot = sr == begin(g) / P.ncc ? 0 : 1;
            v += part[((g * 2 + slot) * rows_per_wg + r) * kBwdSlab + l];
        }
        const int b = m / s.HW, hw = m - b * s.HW;
        GX[x_off(s, b, grp, ci, hw)] = v;
    }
}

// pre-pass: the per-(row, co) factor, transposed to [gco][m]
//   p = 1: grad_output ;  p >= 2: sign(g) * |g|^(1/(p-1)) / out  (root in double precision: its error is multiplied
//   by p-1 when the main kernel raises the factor to that power again) ;  1 < p < 2 (second == 1): 1/out, and
//   grad_output in a second array g_off floats further ;  second == 2 (large exponents): the second array holds
//   what the float32 factor dropped of the double-precision one
__global__ __launch_bounds__(256) void bwd_prepare_kernel(const float* __restrict__ out, const float* __restrict__ gout,
                                                          float* __restrict__ aT, const Geom s, int Mpad, float q, long g_off,
                                                          int second, float* __restrict__ gmax) {
    // tile: 32 rows (m) x 32 columns (gco); reads follow the source's contiguous axis, writes follow m
    __shared__ float ts[32][33], tg[32][33];
    __shared__ float wave_max[4];
    float gmx = 0.f;  // largest |grad_output| this thread has seen
    const int CO = s.COg * s.G;
    const int m0 = blockIdx.x * 32, c0 = blockIdx.y * 32;
    const int tx = threadIdx.x & 31, ty = threadIdx.x >> 5;  // 32 x 8
    // -> the factor; `other` receives the value of the second array
    auto factor = [&](long idx, float& other) -> float {
        const float g = gout[idx];
        other = second == 1 ? g : 0.f;
        gmx = fmaxf(gmx, fabsf(g));
        if (q == 0.f) return g;
        if (second == 1) return 1.0f / out[idx];
        if (g == 0.f) return 0.f;
        // the root in double precision (its relative error is multiplied by q in the terms); exp2(log2 / q) is
        // accurate to a few double ulps and several times cheaper than pow
        const double root = q == 1.f ? (double)fabsf(g) : exp2(log2((double)fabsf(g)) / (double)q);
        const double a = copysign(root, (double)g) / (double)out[idx];
        const float af = (float)a;
        if (second == 2) other = (float)(a - (double)af);
        return af;
    };
    if (s.HW == 1) {
#pragma unroll
        for (int r = ty; r < 32; r += 8) {
            const int m = m0 + r, c = c0 + tx;
            const bool ok = m < s.M && c < CO;
            float o = 0.f;
            ts[r][tx] = ok ? factor((long)m * CO + c, o) : 0.f;
            tg[r][tx] = o;
        }
    } else {
#pragma unroll
        for (int cidx = ty; cidx < 32; cidx += 8) {
            const int m = m0 + tx, c = c0 + cidx;
            float v = 0.f, gv = 0.f;
            if (m < s.M && c < CO) {
                const int b = m / s.HW, hw = m - b * s.HW;
                v = factor(((long)b * CO + c) * s.HW + hw, gv);
            }
            ts[tx][cidx] = v;
            tg[tx][cidx] = gv;
        }
    }
    if (gmax != nullptr) {
#pragma unroll
        for (int d = 32; d >= 1; d >>= 1) gmx = fmaxf(gmx, __shfl_xor(gmx, d, 64));
        if ((threadIdx.x & 63) == 0) wave_max[threadIdx.x >> 6] = gmx;
    }
    __syncthreads();
    if (gmax != nullptr && threadIdx.x == 0) {
        // max|grad_output| of the tile: one atomic per workgroup (non-negative floats order like their bit patterns)
        const float mx = fmaxf(fmaxf(wave_max[0], wave_max[1]), fmaxf(wave_max[2], wave_max[3]));
        if (mx > 0.f) atomicMax(reinterpret_cast<unsigned int*>(gmax), __float_as_uint(mx));
    }
#pragma unroll
    for (int cidx = ty; cidx < 32; cidx += 8) {
        const int m = m0 + tx, c = c0 + cidx;
        if (m < Mpad && c < CO) {
            aT[(long)c * Mpad + m] = ts[tx][cidx];
            if (second != 0) aT[g_off + (long)c * Mpad + m] = tg[tx][cidx];
        }
    }
}

__global__ __launch_bounds__(256) void fill_zero_kernel(float4* __restrict__ p4, long n4, float* __restrict__ tail, int ntail) {
    const long i = (long)blockIdx.x * 256 + threadIdx.x;
    if (i < n4) p4[i] = make_float4(0.f, 0.f, 0.f, 0.f);
    if (i < ntail) tail[i] = 0.f;
}

// zero-fill with a kernel (not a memset node: callers may capture these launches into a graph)
int fill_zero(float* p, long n, hipStream_t st) {
    if (n <= 0) return 0;
    long head = 0;
    while (((uintptr_t)(p + head) % 16) != 0 && head < n) head++;
    const long n4 = (n - head) / 4;
    const long rest = n - head - 4 * n4;
    if (head) hipLaunchKernelGGL(fill_zero_kernel, dim3(1), dim3(256), 0, st, nullptr, 0L, p, (int)head);
    const long blocks = (n4 + 255) / 256 > 0 ? (n4 + 255) / 256 : 1;
    hipLaunchKernelGGL(fill_zero_kernel, dim3((unsigned)blocks), dim3(256), 0, st,
                       reinterpret_cast<float4*>(p + head), n4, p + head + 4 * n4, (int)rest);
    return hip_failed(hipGetLastError()) ? 4 : 0;
}

// batched 2-D transpose: src [batch][R][C] -> dst [batch][C][R], 64 x 64 tiles through LDS, both sides coalesced
__global__ __launch_bounds__(256) void transpose_kernel(const float* __restrict__ src, float* __restrict__ dst, int R,
                                                        int C) {
    __shared__ float tile[64][65];
    const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;
    const int r0 = blockIdx.y * 64, c0 = blockIdx.x * 64;
    const long base = (long)blockIdx.z * R * C;
#pragma unroll
    for (int i = 0; i < 16; i++) {
        const int r = r0 + ty + 4 * i, c = c0 + tx;
        if (r < R && c < C) tile[ty + 4 * i][tx] = src[base + (long)r * C + c];
    }
    __syncthreads();
#pragma unroll
    for (int i = 0; i < 16; i++) {
        const int c = c0 + ty + 4 * i, r = r0 + tx;
        if (r < R && c < C) dst[base + (long)c * R + r] = tile[tx][ty + 4 * i];
    }
}

static int transpose_batched(const float* src, float* dst, int batch, int R, int C, hipStream_t st) {
    if (batch > 65535 || ceil_div(R, 64) > 65535) return 2;
    hipLaunchKernelGGL(transpose_kernel, dim3(ceil_div(C, 64), ceil_div(R, 64), batch), dim3(256), 0, st, src, dst, R, C);
    return hip_failed(hipGetLastError()) ? 4 : 0;
}

// Probe for the choice between the two skipping variants: on a sample of (four rows, co, ci slab) groups, the number
// whose bound |a| (max|x| + max|w|) exceeds the drop threshold, i.e. the groups the bounds variant would still have to
// look at term by term.  One wave per sample; x in the geometry the main kernel will see.
constexpr int kBoundProbeSamples = 4096;
constexpr int kBoundProbeBlock = 1024, kBoundProbePerWave = 4;  // 64 samples per workgroup, one atomic each
__global__ __launch_bounds__(kBoundProbeBlock) void bwd_bound_probe_kernel(const float* __restrict__ x,
                                                                           const float* __restrict__ w,
                                                                           const float* __restrict__ aT, const Geom s,
                                                                           int Mpad, float q, const float* __restrict__ gmax,
                                                                           int* __restrict__ count) {
    constexpr int NWV = kBoundProbeBlock / 64;
    __shared__ int part[NWV];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const float thr = fast_exp2((fast_log2(gmax[0]) - 40.0f) / q);
    const int nslab = ceil_div(s.CIg, kBwdSlab);
    int hits = 0;
    for (int j = 0; j < kBoundProbePerWave; j++) {
        const long i = ((long)blockIdx.x * NWV + wave) * kBoundProbePerWave + j;
        const int g = (int)(i % s.G);
        const int slab = (int)((i * 7919 + 3) % nslab), co = (int)((i * 104729 + 11) % s.COg);
        const int m0 = (int)((i * 1299709 + 5) % ceil_div(s.M, 4)) * 4;
        const int ci = min(slab * kBwdSlab + lane, s.CIg - 1);
        float wm = fabsf(w[w_off(s, g, co, ci)]);
        float xm[4];
#pragma unroll
        for (int r = 0; r < 4; r++) {
            const int m = min(m0 + r, s.M - 1), b = m / s.HW, hw = m - b * s.HW;
            xm[r] = fabsf(x[x_off(s, b, g, ci, hw)]);
        }
#pragma unroll
        for (int d = 32; d >= 1; d >>= 1) {
            wm = fmaxf(wm, __shfl_xor(wm, d, 64));
#pragma unroll
            for (int r = 0; r < 4; r++) xm[r] = fmaxf(xm[r], __shfl_xor(xm[r], d, 64));
        }
        bool hot = false;
#pragma unroll
        for (int r = 0; r < 4; r++) {
            const int m = min(m0 + r, s.M - 1);
            hot |= fabsf(aT[(long)(g * s.COg + co) * Mpad + m]) * (xm[r] + wm) > thr;
        }
        hits += hot ? 1 : 0;  // the same in every lane
    }
    if (lane == 0) part[wave] = hits;
    __syncthreads();
    if (threadIdx.x == 0) {
        int t = 0;
        for (int k = 0; k < NWV; k++) t += part[k];
        if (t != 0) atomicAdd(count, t);
    }
}

// The main kernel spreads ci over the lanes of a wave, which is a coalesced access only when ci is the contiguous
// axis of x (HW == 1).  In the unfolded-conv layout x and grad_x are [B][CI][HW]: from this many positions on they
// are transposed to [B*HW][CI] in scratch memory around the main kernel, which then runs on the fully-connected
// geometry (M rows, HW = 1); the factors are indexed by row in both geometries.
constexpr int kBwdTransposeMinHW = 16;

// What the launcher decides from the shape and the exponent alone.
constexpr float kBwdCompensateFromQ = 64.0f;
struct BwdPlan {
    int ip;              // exponent variant of the kernels
    bool second;         // the variant reads a second factor array
    int cfg;             // 0..2, 4: row-split workgroups of 16 / 8 / 4, 2 waves; 3: small-batch kernel
    int rows_per_wg;
    bool want_adaptive;  // large exponent on a problem worth the probes: skipping and plain variants are all queued
};
static BwdPlan plan_backward(const Geom& s, float p) {
    const float q = p - 1.0f;
    BwdPlan pl{};
    pl.ip = q >= 1.0f ? -1 : -2;  // general exponent; below 1 grad_output is not folded into the factor
    if (q == (float)(int)q && (int)q >= 0 && (int)q <= 8) pl.ip = (int)q;  // as far as the reference's ladder goes
    // 3: small-batch kernel (waves split co, 32-row chunks); its grid index must fit 32 bits
    const bool small = s.M <= kBwdSmallMaxM && (long)s.G * ceil_div(s.CIg, kBwdSlab) * ceil_div(s.M, kBwdSmallRows) * 64 < (1L << 31);
    // Large exponents on problems worth the extra launches: the skipping variants (IP -3, -4) and the plain one
    // (IP -1) are all queued and device-side probes of the data open the gate of one of them.
    pl.want_adaptive = pl.ip == -1 && q >= 15.0f && ((double)s.M * s.COg * s.G * s.CIg >= 2e8 || skip_forced_on());
    // large exponents: the product under the power is compensated (see bwd_terms), the pre-pass writes what every
    // float32 factor dropped into a second array
    if (pl.ip == -1 && q >= kBwdCompensateFromQ) pl.ip = -5;
    pl.second = pl.ip == -2 || pl.ip == -5;
    pl.cfg = 3;
    if (!small) {
        // rows are padded to whole chunks of a workgroup's rows (512, 256 or 128): the configuration with the least
        // padded work wins; measured cost of one chunk relative to the 512-row one: 1, 0.505, 0.28.  The bounds
        // variant of the large exponents costs per chunk rather than per row (1, 0.75, 0.6: it spends its time on
        // the weights and factors of a unit, not on the rows); which variant will run is not known here, so the
        // large exponents use the mean of the two cost vectors.
        // With few output columns the rows change every few units, and a workgroup's waves then all wait for the new
        // rows together: two 8-wave workgroups per compute unit cover each other's waits, one of 16 waves cannot
        // (3 x 3 conv, 128 channels: 3 - 6 % faster at 64 ... 512 output columns, 0 - 7 % slower at 1024).
        constexpr double kChunkCost[2][3] = {{1.0, 0.505, 0.28}, {1.0, 0.63, 0.44}};
        const bool few_columns = ceil_div(s.COg, kBwdCoUnit) <= 32;
        double best = 0.0;
        for (int c = 0; c < 3; c++) {
            double cost = kChunkCost[pl.want_adaptive ? 1 : 0][c] * ceil_div(s.M, kBwdCfgRows[c] * kBwdCfgWaves[c]);
            if (c == 1 && few_columns && !pl.want_adaptive) cost *= 0.94;
            if (c == 0 || cost < best) { best = cost; pl.cfg = c; }
        }
        if (s.M <= 64) pl.cfg = 4;  // one 64-row chunk (0.33 ms at 5120 x 5120 against 0.51 for a 128-row chunk)
        // tuning aid: NORM_DIST_BWD_CFG=0 / 1 / 2 forces the 16- / 8- / 4-wave workgroups
        static const char* force = getenv("NORM_DIST_BWD_CFG");
        if (force != nullptr && force[0] >= '0' && force[0] <= '2') pl.cfg = force[0] - '0';
    }
    pl.rows_per_wg = small ? bwd_small_rows(s.M) : kBwdCfgRows[pl.cfg] * kBwdCfgWaves[pl.cfg];
    return pl;
}

// the description of the images goes to device memory through a kernel, so that it is part of a captured graph
__global__ void bwd_image_kernel(const BwdImage v, BwdImage* __restrict__ dst) {
    if (threadIdx.x == 0) *dst = v;
}

// NORM_DIST_BWD_GATHER=0: the patches of a conv layer are always written out as rows first (the path of the
// skipping variants and of small batches); read at every call
static bool bwd_gather_enabled() {
    const char* e = getenv("NORM_DIST_BWD_GATHER");
    return e == nullptr || e[0] != '0';
}

bool norm_backward_gathers(const Geom& s, float p) {
    const BwdPlan pl = plan_backward(s, p);
    return !pl.want_adaptive && pl.cfg != 3 && bwd_gather_enabled();
}

size_t norm_backward_scratch_bytes(const Geom& s, float p) {
    const BwdPlan pl = plan_backward(s, p);
    const size_t mpad = (size_t)ceil_div(s.M, pl.rows_per_wg) * pl.rows_per_wg;
    return (size_t)s.COg * s.G * mpad * sizeof(float) * (pl.second ? 2 : 1);
}

int launch_norm_backward(const float* gout, const float* x, const float* w, const float* out, const Geom& s, float* gx,
                         float* gw, float p, hipStream_t st, const UnfoldGeom* cv, bool gw_accumulate) {
    const float q = p - 1.0f;
    const BwdPlan pl = plan_backward(s, p);
    const int ip = pl.ip, cfg = pl.cfg;
    const bool want_adaptive = pl.want_adaptive;
    const int rows_per_wg = pl.rows_per_wg;

    BwdParams P{};
    P.s = s;
    P.nrc = ceil_div(s.M, rows_per_wg);
    P.Mpad = P.nrc * rows_per_wg;
    P.nslab = ceil_div(s.CIg, kBwdSlab);
    P.ncc = ceil_div(s.COg, kBwdCoUnit);
    P.total = (long)s.G * P.nslab * P.nrc * P.ncc;
    P.q = q;
    P.gw_add = P.nrc > 1 || gw_accumulate ? 1 : 0;

    const size_t tbytes = (size_t)s.COg * s.G * P.Mpad * sizeof(float);
    float* aT = nullptr;
    P.g_off = pl.second ? (long)s.COg * s.G * P.Mpad : 0;
    NDIST_HIP_TRY(scratch_alloc((void**)&aT, pl.second ? 2 * tbytes : tbytes, st));

    int rc = 0;
    // (thin upper tail of |x - w|: skipping is up to twice as fast; many pairs near the maximum: it would be slower)
    bool adaptive = want_adaptive;
    float* aux = nullptr;  // [0]: probe count (int), [1]: count of the bounds probe (int), [4]: max|grad_output|
    if (adaptive && scratch_alloc((void**)&aux, 32, st) != hipSuccess) {
        (void)hipGetLastError();  // the plain variant needs no scratch
        aux = nullptr;
        adaptive = false;
    }
    if (adaptive) {
        rc = fill_zero(aux, 8, st);
        // (on images the probe runs below, on the patch rows)
        if (!rc && cv == nullptr) rc = launch_norm_probe(x, w, s, exp2f(-40.0f / q), reinterpret_cast<int*>(aux), st);
        P.gmax = aux + 4;
        P.gate = reinterpret_cast<const int*>(aux);
        P.gate_limit = skip_override_limit(norm_probe_limit(s));
    }
    if (!rc) {
        dim3 grid(ceil_div(P.Mpad, 32), ceil_div(s.COg * s.G, 32));
        hipLaunchKernelGGL(bwd_prepare_kernel, grid, dim3(256), 0, st, out, gout, aT, s, P.Mpad, q, P.g_off,
                           ip == -2 ? 1 : (pl.second ? 2 : 0), adaptive ? aux + 4 : (float*)nullptr);
        if (hip_failed(hipGetLastError())) rc = 4;
    }
    const long nx = (long)s.M * s.CIg * s.G;
    // On images (cv): the patches are written straight into the row layout (or, for geometries that kernel does not
    // take, extracted into a third buffer in the unfolded layout [B][CI][HW] and transposed like an unfolded input);
    // the gradient rows are folded back into the image by one gather.
    bool transposed = cv != nullptr || (s.HW >= kBwdTransposeMinHW && s.B <= 65535);
    float* xT = nullptr;  // [M][CI] copy of x, followed by the [M][CI] gradient (and the unfolded buffer)
    float* unfolded = nullptr;
    // The main kernel gathers the patches from the images itself (BwdParams::img): no copy of x in the row layout,
    // only the gradient rows.  (The probes of the skipping variants and the small-batch kernel read rows.)
    const bool gather = cv != nullptr && !want_adaptive && cfg != 3 && bwd_gather_enabled();
    if (!rc && gather) {
        const hipError_t e = scratch_alloc((void**)&xT, (size_t)nx * sizeof(float), st);
        if (e != hipSuccess) {
            (void)scratch_free(aT, st);
            return hip_status(e);
        }
        P.s.B = s.M;
        P.s.HW = 1;
        BwdImage* image = nullptr;
        const hipError_t e2 = scratch_alloc((void**)&image, sizeof(BwdImage), st);
        if (e2 != hipSuccess) {
            (void)scratch_free(xT, st);
            (void)scratch_free(aT, st);
            return hip_status(e2);
        }
        hipLaunchKernelGGL(bwd_image_kernel, dim3(1), dim3(64), 0, st, BwdImage{x, *cv}, image);
        if (hip_failed(hipGetLastError())) rc = 4;
        P.image = image;
    } else if (!rc && transposed) {
        const bool via_unfold = cv != nullptr && !patch_rows_applies(*cv);  // needs the third buffer
        const hipError_t e = scratch_alloc((void**)&xT, (via_unfold ? 3 : 2) * (size_t)nx * sizeof(float), st);
        if (e != hipSuccess && cv != nullptr) {  // on images there is no other path
            if (aux != nullptr) (void)scratch_free(aux, st);
            (void)scratch_free(aT, st);
            return hip_status(e);
        }
        if (e != hipSuccess) {
            (void)hipGetLastError();  // no room for the copies: the direct, uncoalesced path still works
            xT = nullptr;
            transposed = false;
        } else {
            const float* src = x;
            bool rows_done = false;
            if (cv != nullptr && !via_unfold) {
                rc = launch_patch_rows(x, *cv, xT, st);  // straight into the row layout
                rows_done = true;
            } else if (cv != nullptr) {
                unfolded = xT + 2 * nx;
                rc = launch_unfold(x, *cv, unfolded, st);
                src = unfolded;
            }
            if (!rc && !rows_done) rc = transpose_batched(src, xT, s.B, s.CIg * s.G, s.HW, st);
            P.s.B = s.M;
            P.s.HW = 1;
            if (!rc && adaptive && cv != nullptr)
                rc = launch_norm_probe(xT, w, P.s, exp2f(-40.0f / q), reinterpret_cast<int*>(aux), st);
        }
    }
    float* gx_k = gather ? xT : (transposed ? xT + nx : gx);
    // Reproducible grad_input: shares of the blocks that two workgroups split go through a buffer and are added in a
    // fixed order (see BwdParams::part).  Not for the small-batch kernel, not where several kernel variants are
    // queued (their grids may differ), not from the fixed scratch array (64 MB at the headline shape): those add
    // with atomics into a zeroed gradient.
    const long cap = (long)device_info().num_cu * (cfg == 1 ? 2 : (cfg == 2 ? 4 : (cfg == 4 ? 6 : 1)));
    const int grid = (int)(P.total < cap ? P.total : cap);
    float* part = nullptr;
    // (NORM_DIST_BWD_ATOMIC=1: tuning aid, the atomic adds everywhere)
    static const bool force_atomic = getenv("NORM_DIST_BWD_ATOMIC") != nullptr && getenv("NORM_DIST_BWD_ATOMIC")[0] == '1';
    if (!rc && cfg != 3 && !adaptive && !static_scratch_active() && !force_atomic) {
        if (scratch_alloc((void**)&part, 2 * (size_t)grid * rows_per_wg * kBwdSlab * sizeof(float), st) != hipSuccess) {
            (void)hipGetLastError();
            part = nullptr;
        }
    }
    P.part = part;
    if (!rc && part == nullptr) rc = fill_zero(gx_k, nx, st);
    if (!rc && gw != nullptr && P.nrc > 1 && !gw_accumulate) rc = fill_zero(gw, (long)s.COg * s.G * s.CIg, st);
    if (!rc) {
        // Persistent workgroups take equal shares of the units, so all of them should be resident at once: two 8-wave
        // workgroups fit a compute unit (72 KB of LDS each), four 4-wave ones (40 KB each, exactly the 160 KB) and six
        // 2-wave ones (24.6 KB each).
        BwdPtrs a{transposed ? xT : x, w, aT, gx_k, gw};
        switch (ip) {
            case 0: rc = launch_bwd_ip<0>(a, P, cfg, grid, st); break;
            case 1: rc = launch_bwd_ip<1>(a, P, cfg, grid, st); break;
            case 2: rc = launch_bwd_ip<2>(a, P, cfg, grid, st); break;
            case 3: rc = launch_bwd_ip<3>(a, P, cfg, grid, st); break;
            case 4: rc = launch_bwd_ip<4>(a, P, cfg, grid, st); break;
            case 5: rc = launch_bwd_ip<5>(a, P, cfg, grid, st); break;
            case 6: rc = launch_bwd_ip<6>(a, P, cfg, grid, st); break;
            case 7: rc = launch_bwd_ip<7>(a, P, cfg, grid, st); break;
            case 8: rc = launch_bwd_ip<8>(a, P, cfg, grid, st); break;
            case -2: rc = launch_bwd_ip<-2>(a, P, cfg, grid, st); break;
            default:
                if (adaptive) {
                    // Three candidates, one runs: plain, skipping term by term, skipping by bounds first.  The second
                    // probe samples the groups of four rows the bounds variant could NOT dismiss; that variant pays
                    // while they are a minority.
                    const bool two = cfg <= 2;  // the bounds variant exists for the row-split configurations
                    int* count2 = reinterpret_cast<int*>(aux) + 1;
                    if (two) {
                        hipLaunchKernelGGL(bwd_bound_probe_kernel,
                                           dim3(kBoundProbeSamples / (kBoundProbeBlock / 64 * kBoundProbePerWave)),
                                           dim3(kBoundProbeBlock), 0, st, a.x, a.w,
                                           a.aT, P.s, P.Mpad, q, aux + 4, count2);
                        if (hip_failed(hipGetLastError())) rc = 4;
                        P.gate2 = count2;
                        P.gate2_limit = bounds_override_limit((int)(0.3 * kBoundProbeSamples));
                    }
                    KernelTimer timer(st);  // whichever of the three runs
                    P.gate_sense = 1;
                    if (!rc && two) {
                        P.gate2_sense = 1;
                        rc = launch_bwd_ip<-4>(a, P, cfg, grid, st);
                        P.gate2_sense = 0;
                    }
                    if (!rc) rc = launch_bwd_ip<-3>(a, P, cfg, grid, st);
                    P.gate2 = nullptr;
                    P.gate_sense = 0;
                    if (!rc) rc = ip == -5 ? launch_bwd_ip<-5>(a, P, cfg, grid, st) : launch_bwd_ip<-1>(a, P, cfg, grid, st);
                } else {
                    rc = ip == -5 ? launch_bwd_ip<-5>(a, P, cfg, grid, st) : launch_bwd_ip<-1>(a, P, cfg, grid, st);
                }
                break;
        }
    }
    if (!rc && part != nullptr) {
        const long nblk = (long)(grid - 1) * ((rows_per_wg * kBwdSlab + 1023) / 1024);
        if (nblk > 0) {
            hipLaunchKernelGGL(bwd_gx_fixup_kernel, dim3((unsigned)nblk), dim3(256), 0, st, part, gx_k, P, grid, rows_per_wg);
            if (hip_failed(hipGetLastError())) rc = 4;
        }
    }
    if (part != nullptr && hip_failed(scratch_free(part, st)) && !rc) rc = 4;
    if (!rc && cv != nullptr) rc = launch_fold_rows(gx_k, *cv, gx, st);
    else if (!rc && transposed) rc = transpose_batched(gx_k, gx, s.B, s.HW, s.CIg * s.G, st);
    if (P.image != nullptr && hip_failed(scratch_free(const_cast<BwdImage*>(P.image), st)) && !rc) rc = 4;
    if (xT != nullptr && hip_failed(scratch_free(xT, st)) && !rc) rc = 4;
    if (aux != nullptr && hip_failed(scratch_free(aux, st)) && !rc) rc = 4;
    if (hip_failed(scratch_free(aT, st)) && !rc) rc = 4;
    return rc;
}

}  // namespace ndist
