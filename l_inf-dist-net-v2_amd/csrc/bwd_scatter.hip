// Backward of the infinity distance and of its interval bounds: every output sends +-grad_output to the one input
// (and weight) position its arg-max code names.  Replaces inf_dist::backward_input[_weight] and
// bound_inf_dist::backward_input[_weight] of the reference (core/cuda/inf_dist_cuda.cu:200-246,319-346;
// core/cuda/bound_inf_dist_cuda.cu:240-299,362-383).
//
// The work is pure memory traffic.  Three paths:
//   * privatised rows (fully-connected layout, HW == 1, rows that fit in LDS): one workgroup owns whole rows of a
//     gradient, accumulates the scattered values in LDS (ds_add_f32) and writes each row once, coalesced; no zero
//     fill, no global atomics.  grad_input rows are indexed by b, grad_weight rows by co.
//   * privatised tiles (unfolded-conv layout, HW > 1): grad_input is produced in LDS tiles of (ci slab) x (16
//     consecutive positions) of one sample, filled from the codes of every co at those positions and written
//     once; grad_weight rows are accumulated in LDS over a share of the batch and added to global memory once per
//     workgroup.
//   * generic: zero-fill kernel followed by global atomic adds, any layout.
//   * images (convolutional layer called with a patch geometry): grad_input is the image gradient itself; a
//     workgroup owns a slab of image channels of one sample in LDS, maps every code of that sample back through the
//     patch geometry (taps in the padding are dropped, as the adjoint of the patch extraction would drop them) and
//     writes the slab once.  The unfolded gradient never exists.
#include "ndist_common.h"
#include "rescan_image.h"

namespace ndist {

int fill_zero(float* p, long n, hipStream_t st);  // bwd_norm_c.hip

// Decoded contribution of one output of the plain infinity distance.
struct Route {
    int idx;     // position inside the group
    float v;     // value added to grad_input (its negative goes to grad_weight)
    int target;  // 0: first input gradient (grad_input / grad_inputL), 1: grad_inputU, -1: nothing
};

__device__ __forceinline__ Route route_inf(int32_t pos, float g) {
    Route r;
    r.idx = (int)((uint32_t)pos & ~kSignBit);
    r.v = pos >= 0 ? g : -g;
    r.target = 0;
    return r;
}
// lower output bound: sign 0 -> grad_xL += g ; sign 1 -> grad_xU -= g ; code 0xffffffff -> nothing
__device__ __forceinline__ Route route_lower(int32_t pos, float g) {
    Route r = route_inf(pos, g);
    r.target = (uint32_t)pos == kNoGradId ? -1 : (pos >= 0 ? 0 : 1);
    return r;
}
// upper output bound: sign 0 -> grad_xU += g ; sign 1 -> grad_xL -= g
__device__ __forceinline__ Route route_upper(int32_t pos, float g) {
    Route r = route_inf(pos, g);
    r.target = pos >= 0 ? 1 : 0;
    return r;
}

// ---- generic path ---------------------------------------------------------------------------------------
template <bool BOUND>
__global__ __launch_bounds__(256) void scatter_atomic_kernel(const float* __restrict__ g1, const float* __restrict__ g2,
                                                             const int32_t* __restrict__ p1,
                                                             const int32_t* __restrict__ p2, float* __restrict__ gx1,
                                                             float* __restrict__ gx2, float* __restrict__ gw,
                                                             const Geom s, long total) {
    const long o = (long)blockIdx.x * 256 + threadIdx.x;
    if (o >= total) return;
    const int hw = (int)(o % s.HW);
    const long r = o / s.HW;
    const int gco = (int)(r % (s.COg * s.G));
    const int b = (int)(r / (s.COg * s.G));
    const int g = gco / s.COg, co = gco - g * s.COg;
    Route rt[2];
    rt[0] = BOUND ? route_lower(p1[o], g1[o]) : route_inf(p1[o], g1[o]);
    if (BOUND) rt[1] = route_upper(p2[o], g2[o]);
#pragma unroll
    for (int q = 0; q < (BOUND ? 2 : 1); q++) {
        if (rt[q].target < 0 || rt[q].idx >= s.CIg) continue;  // a corrupt code must not become a wild store
        float* dst = rt[q].target == 0 ? gx1 : gx2;
        atomicAdd(dst + x_off(s, b, g, rt[q].idx, hw), rt[q].v);
        if (gw) atomicAdd(gw + w_off(s, g, co, rt[q].idx), -rt[q].v);
    }
}

// LDS float add of one value per lane, with the lanes of a wave that target the same word combined first.  Codes
// cluster: every output of a batch row whose largest |x| dominates names the same input, every batch row of an
// output whose weight row has one dominant entry names the same weight, and thousands of adds to one LDS word
// serialise.  At most two clusters of eight or more lanes are summed across the wave (butterfly) and added once by
// their first lane; what remains goes through plain adds.  off < 0: the lane has nothing to add.
template <int CTRL>
__device__ __forceinline__ float dpp_add(float v) {
    return v + __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xf, 0xf, true));
}
// Sum over the 64 lanes of a wave (all active), the same value in every lane: butterfly inside the quads
// (quad_perm [1,0,3,2], [2,3,0,1]), rotations by 4 and 8 inside the rows of 16, then the four row sums.
__device__ __forceinline__ float wave_sum(float v) {
    v = dpp_add<0xB1>(v);
    v = dpp_add<0x4E>(v);
    v = dpp_add<0x124>(v);
    v = dpp_add<0x128>(v);
    const int i = __builtin_bit_cast(int, v);
    return (__builtin_bit_cast(float, __builtin_amdgcn_readlane(i, 0)) + __builtin_bit_cast(float, __builtin_amdgcn_readlane(i, 16))) +
           (__builtin_bit_cast(float, __builtin_amdgcn_readlane(i, 32)) + __builtin_bit_cast(float, __builtin_amdgcn_readlane(i, 48)));
}
template <typename ACC>
__device__ __forceinline__ void lds_add_clustered(ACC* base, int off, float v) {
    const int lane = threadIdx.x & 63;
    bool active = off >= 0;
#pragma unroll 1
    for (int round = 0; round < 2; round++) {
        const unsigned long long todo = __builtin_amdgcn_ballot_w64(active);
        if (todo == 0) return;
        const int leader = __builtin_ctzll(todo);
        const int loff = __builtin_amdgcn_readlane(off, leader);
        const bool mine = active && off == loff;
        const unsigned long long grp = __builtin_amdgcn_ballot_w64(mine);
        if (__builtin_popcountll(grp) < 8) break;
        const float sum = wave_sum(mine ? v : 0.f);
        if (lane == leader) atomicAdd(base + loff, (ACC)sum);
        active = active && !mine;
    }
    if (active) atomicAdd(base + off, (ACC)v);
}

constexpr int kScatterBatch = 8;  // outputs whose codes and gradients a thread requests before it adds any of them

// ---- privatised path, HW == 1 ---------------------------------------------------------------------------
// grad_input: one workgroup per (b, g); LDS holds the CIg-long row (two rows for the interval variant).
// ACC: float, or double (LDS double adds run at nine times the rate of float ones on this part, see below).
template <bool BOUND, typename ACC>
__global__ __launch_bounds__(1024) void scatter_gx_rows_kernel(const float* __restrict__ g1, const float* __restrict__ g2,
                                                              const int32_t* __restrict__ p1,
                                                              const int32_t* __restrict__ p2, float* __restrict__ gx1,
                                                              float* __restrict__ gx2, const Geom s) {
    extern __shared__ __align__(16) float row_lds[];
    ACC* __restrict__ row = reinterpret_cast<ACC*>(row_lds);  // [BOUND ? 2 : 1][CIg]
    const int b = blockIdx.x, g = blockIdx.y, nt = blockDim.x;
    const int nrow = (BOUND ? 2 : 1) * s.CIg;
    const long xbase = x_off(s, b, g, 0, 0);
    // 16-byte LDS and global accesses when the rows allow it (the dynamic LDS base is 16-byte aligned)
    const bool vec = s.CIg % 4 == 0 && (uintptr_t)(gx1 + xbase) % 16 == 0 && (!BOUND || (uintptr_t)(gx2 + xbase) % 16 == 0);
    for (int i = threadIdx.x; i < nrow; i += nt) row[i] = (ACC)0;
    __syncthreads();
    const long obase = y_off(s, b, g, 0, 0);
    // the loads of kScatterBatch outputs are issued together: one memory latency per batch, not per output
    // (the loop bounds are the same for all threads: lds_add_clustered needs whole waves)
    for (int k0 = 0; k0 < s.COg; k0 += nt * kScatterBatch) {
        const int c0 = k0 + threadIdx.x;
        int32_t pa[kScatterBatch], pb[kScatterBatch];
        float ga[kScatterBatch], gb[kScatterBatch];
#pragma unroll
        for (int u = 0; u < kScatterBatch; u++) {
            const int co = min(c0 + u * nt, s.COg - 1);  // clamped, not guarded: no branch between the loads
            pa[u] = p1[obase + co];
            ga[u] = g1[obase + co];
            if (BOUND) {
                pb[u] = p2[obase + co];
                gb[u] = g2[obase + co];
            }
        }
#pragma unroll
        for (int u = 0; u < kScatterBatch; u++) {
            if (k0 + u * nt < s.COg) {  // some thread of this step has an output
                const bool live = c0 + u * nt < s.COg;
                const Route a = BOUND ? route_lower(pa[u], ga[u]) : route_inf(pa[u], ga[u]);
                lds_add_clustered(row, live && a.target >= 0 && a.idx < s.CIg ? a.target * s.CIg + a.idx : -1, a.v);
                if (BOUND) {
                    const Route c = route_upper(pb[u], gb[u]);
                    lds_add_clustered(row, live && c.idx < s.CIg ? c.target * s.CIg + c.idx : -1, c.v);
                }
            }
        }
    }
    __syncthreads();
    if (vec) {
        auto sum4 = [&](int e) { return make_float4((float)row[e], (float)row[e + 1], (float)row[e + 2], (float)row[e + 3]); };
        for (int i = threadIdx.x; i < s.CIg / 4; i += nt) {
            reinterpret_cast<float4*>(gx1 + xbase)[i] = sum4(4 * i);
            if (BOUND) reinterpret_cast<float4*>(gx2 + xbase)[i] = sum4(s.CIg + 4 * i);
        }
    } else {
        for (int i = threadIdx.x; i < s.CIg; i += nt) {
            gx1[xbase + i] = (float)row[i];
            if (BOUND) gx2[xbase + i] = (float)row[s.CIg + i];
        }
    }
}

// grad_weight: one workgroup per R consecutive rows (co) of one group; LDS holds R rows of CIg.
template <bool BOUND>
__global__ __launch_bounds__(256) void scatter_gw_rows_kernel(const float* __restrict__ g1, const float* __restrict__ g2,
                                                              const int32_t* __restrict__ p1,
                                                              const int32_t* __restrict__ p2, float* __restrict__ gw,
                                                              const Geom s, int R) {
    extern __shared__ float rows[];  // [R][CIg]
    // Workgroups are handed to the eight XCDs in turn, and a workgroup uses 4 R bytes of every 128-byte line of
    // grad_output and codes it touches: numbered as launched, the neighbours that share its lines would sit on
    // the other seven XCDs and every L2 would fetch every line.  Renumbered so that each XCD owns a contiguous
    // range of co blocks, the workgroups resident on one XCD share the lines.
    int g, cb;
    {
        const int total = gridDim.x * gridDim.y, id = blockIdx.y * gridDim.x + blockIdx.x;
        const int q = total / 8, rem = total % 8, xcd = id % 8, slot = id / 8;
        const int logical = xcd * q + min(xcd, rem) + slot;
        g = logical / gridDim.x;
        cb = logical - g * gridDim.x;
    }
    const int co0 = cb * R;
    const int nr = min(R, s.COg - co0);
    float* dst = gw + w_off(s, g, co0, 0);
    const bool vec = s.CIg % 4 == 0 && (uintptr_t)dst % 16 == 0;
    if (vec) {
        for (int i = threadIdx.x; i < nr * s.CIg / 4; i += 256) reinterpret_cast<float4*>(rows)[i] = make_float4(0.f, 0.f, 0.f, 0.f);
    } else {
        for (int i = threadIdx.x; i < nr * s.CIg; i += 256) rows[i] = 0.f;
    }
    __syncthreads();
    // thread -> (b, r): r fastest so that one b's R codes are read as one contiguous segment
    const int n = s.B * nr;
    for (int i0 = 0; i0 < n; i0 += 256) {
        const int i = i0 + threadIdx.x;
        const bool live = i < n;
        const int b = live ? i / nr : 0, r = live ? i - b * nr : 0;
        const long o = y_off(s, b, g, co0 + r, 0);
        const Route a = BOUND ? route_lower(p1[o], g1[o]) : route_inf(p1[o], g1[o]);
        lds_add_clustered(rows, live && a.target >= 0 && a.idx < s.CIg ? r * s.CIg + a.idx : -1, -a.v);
        if (BOUND) {
            const Route c = route_upper(p2[o], g2[o]);
            lds_add_clustered(rows, live && c.idx < s.CIg ? r * s.CIg + c.idx : -1, -c.v);
        }
    }
    __syncthreads();
    if (vec) {
        for (int i = threadIdx.x; i < nr * s.CIg / 4; i += 256) reinterpret_cast<float4*>(dst)[i] = reinterpret_cast<const float4*>(rows)[i];
    } else {
        for (int i = threadIdx.x; i < nr * s.CIg; i += 256) dst[i] = rows[i];
    }
}


// ---- privatised path, HW > 1 ----------------------------------------------------------------------------
constexpr int kScatterHB = 16;  // consecutive positions per grad_input tile: 64-byte segments of every row

// grad_input: one workgroup per (b, g, block of 16 positions, ci slab of CS).  LDS holds [BOUND ? 2 : 1][CS][16].
// Adjacent lanes read the codes of adjacent positions of one co; codes outside the slab are skipped.
template <bool BOUND>
__global__ __launch_bounds__(256) void scatter_gx_tile_kernel(const float* __restrict__ g1, const float* __restrict__ g2,
                                                              const int32_t* __restrict__ p1,
                                                              const int32_t* __restrict__ p2, float* __restrict__ gx1,
                                                              float* __restrict__ gx2, const Geom s, int CS, int nslab,
                                                              int nhb) {
    extern __shared__ float tile[];
    constexpr int HB = kScatterHB;
    unsigned id = blockIdx.x;
    const int slab = (int)(id % (unsigned)nslab);
    id /= (unsigned)nslab;
    const int hb = (int)(id % (unsigned)nhb);
    id /= (unsigned)nhb;
    const int g = (int)(id % (unsigned)s.G), b = (int)(id / (unsigned)s.G);
    const int c0 = slab * CS, cs = min(CS, s.CIg - c0), hw0 = hb * HB;
    const int ntile = (BOUND ? 2 : 1) * CS * HB;
    for (int i = threadIdx.x; i < ntile; i += 256) tile[i] = 0.f;
    __syncthreads();
    const int h = threadIdx.x & (HB - 1), hw = hw0 + h;
    if (hw < s.HW) {
        for (int co = threadIdx.x / HB; co < s.COg; co += 256 / HB) {
            const long o = y_off(s, b, g, co, hw);
            const Route a = BOUND ? route_lower(p1[o], g1[o]) : route_inf(p1[o], g1[o]);
            const unsigned ka = (unsigned)(a.idx - c0);
            if (a.target >= 0 && ka < (unsigned)cs) atomicAdd(tile + ((long)a.target * CS + ka) * HB + h, a.v);
            if (BOUND) {
                const Route c = route_upper(p2[o], g2[o]);
                const unsigned kc = (unsigned)(c.idx - c0);
                if (kc < (unsigned)cs) atomicAdd(tile + ((long)c.target * CS + kc) * HB + h, c.v);
            }
        }
    }
    __syncthreads();
    const long xbase = x_off(s, b, g, c0, hw0);
    if (s.HW % 4 == 0 && (uintptr_t)gx1 % 16 == 0 && (!BOUND || (uintptr_t)gx2 % 16 == 0)) {
        // hw0 is a multiple of 16 and HW of 4: whole quads are inside or outside the row
        for (int i = threadIdx.x; i < cs * (HB / 4); i += 256) {
            const int k = i / (HB / 4), q = (i % (HB / 4)) * 4;
            if (hw0 + q < s.HW) {
                *reinterpret_cast<float4*>(gx1 + xbase + (long)k * s.HW + q) =
                    *reinterpret_cast<const float4*>(tile + k * HB + q);
                if (BOUND)
                    *reinterpret_cast<float4*>(gx2 + xbase + (long)k * s.HW + q) =
                        *reinterpret_cast<const float4*>(tile + (CS + k) * HB + q);
            }
        }
    } else {
        for (int i = threadIdx.x; i < cs * HB; i += 256) {
            const int k = i / HB, q = i % HB;
            if (hw0 + q < s.HW) {
                gx1[xbase + (long)k * s.HW + q] = tile[k * HB + q];
                if (BOUND) gx2[xbase + (long)k * s.HW + q] = tile[(CS + k) * HB + q];
            }
        }
    }
}

// grad_weight: one workgroup per (R consecutive co of one group, share of the batch); LDS holds R rows of CIg.
// With one share the rows are stored, with several they are added to the zero-filled gradient.
template <bool BOUND>
__global__ __launch_bounds__(256) void scatter_gw_split_kernel(const float* __restrict__ g1, const float* __restrict__ g2,
                                                               const int32_t* __restrict__ p1,
                                                               const int32_t* __restrict__ p2, float* __restrict__ gw,
                                                               const Geom s, int R, int nsplit) {
    extern __shared__ float rows[];  // [R][CIg]
    const int g = blockIdx.y, co0 = blockIdx.x * R, j = blockIdx.z;
    const int nr = min(R, s.COg - co0);
    const int b0 = (int)((long)j * s.B / nsplit), b1 = (int)((long)(j + 1) * s.B / nsplit);
    for (int i = threadIdx.x; i < nr * s.CIg; i += 256) rows[i] = 0.f;
    __syncthreads();
    // thread -> (b, r, hw), hw fastest: the codes of one (b, co) are one contiguous run
    const long total = (long)(b1 - b0) * nr * s.HW;
    for (long i = threadIdx.x; i < total; i += 256) {
        const int hw = (int)(i % s.HW);
        const int t = (int)(i / s.HW);
        const int r = t % nr, b = b0 + t / nr;
        const long o = y_off(s, b, g, co0 + r, hw);
        const Route a = BOUND ? route_lower(p1[o], g1[o]) : route_inf(p1[o], g1[o]);
        if (a.target >= 0 && a.idx < s.CIg) atomicAdd(rows + r * s.CIg + a.idx, -a.v);
        if (BOUND) {
            const Route c = route_upper(p2[o], g2[o]);
            if (c.idx < s.CIg) atomicAdd(rows + r * s.CIg + c.idx, -c.v);
        }
    }
    __syncthreads();
    float* dst = gw + w_off(s, g, co0, 0);
    if (nsplit == 1) {
        for (int i = threadIdx.x; i < nr * s.CIg; i += 256) dst[i] = rows[i];
    } else {
        for (int i = threadIdx.x; i < nr * s.CIg; i += 256)
            if (rows[i] != 0.f) atomicAdd(dst + i, rows[i]);
    }
}

// ---- sums in double precision ---------------------------------------------------------------------------------
// An LDS float add (ds_add_f32) takes about 190 cycles per wave instruction on this part, a double one (ds_add_f64)
// 21, a 64-bit integer one 11 (measured on random words).  Where a workgroup's sums live in LDS and the adds do not
// pile up on few words, it therefore adds doubles and rounds once at the end: nine times the rate, and sums that are
// exact to far below float precision whatever the order of the adds (infinities and NaNs travel as they do in
// floats).  The price is eight bytes of LDS per sum.

// grad_weight as scatter_gw_split_kernel, sums in doubles.  LDS: [R][CIg] doubles.  1024 threads: as many waves per
// compute unit from a quarter of the workgroups, i.e. a quarter of the adds to global memory at the end.
constexpr int kGwWideThreads = 1024;
template <bool BOUND>
__global__ __launch_bounds__(kGwWideThreads) void scatter_gw_split_f64_kernel(const float* __restrict__ g1, const float* __restrict__ g2,
                                                                              const int32_t* __restrict__ p1,
                                                                              const int32_t* __restrict__ p2, float* __restrict__ gw,
                                                                              const Geom s, int R, int nsplit) {
    extern __shared__ double acc[];  // [R][CIg]
    const int g = blockIdx.y, co0 = blockIdx.x * R, j = blockIdx.z;
    const int nr = min(R, s.COg - co0);
    const int b0 = (int)((long)j * s.B / nsplit), b1 = (int)((long)(j + 1) * s.B / nsplit);
    for (int i = threadIdx.x; i < nr * s.CIg; i += kGwWideThreads) acc[i] = 0.0;
    __syncthreads();
    // A wave takes whole runs -- the HW outputs of one (b, co), contiguous in memory -- with its lanes along hw, and
    // requests the loads of U steps of 64 outputs together: the waves would otherwise wait one memory latency per
    // step, and no index needs a division per output.
    constexpr int U = 8;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nwave = kGwWideThreads / 64;
    const int nrun = (b1 - b0) * nr;
    for (int t = wave; t < nrun; t += nwave) {
        const int r = t % nr;
        const long o0 = y_off(s, b0 + t / nr, g, co0 + r, 0);
        for (int h0 = 0; h0 < s.HW; h0 += 64 * U) {
            float ga[U], gb[U];
            int32_t pa[U], pb[U];
#pragma unroll
            for (int u = 0; u < U; u++) {
                const int hw = min(h0 + 64 * u + lane, s.HW - 1);
                ga[u] = g1[o0 + hw];
                pa[u] = p1[o0 + hw];
                if (BOUND) {
                    gb[u] = g2[o0 + hw];
                    pb[u] = p2[o0 + hw];
                }
            }
#pragma unroll
            for (int u = 0; u < U; u++) {
                if (h0 + 64 * u + lane >= s.HW) continue;
                const Route a = BOUND ? route_lower(pa[u], ga[u]) : route_inf(pa[u], ga[u]);
                if (a.target >= 0 && a.idx < s.CIg) atomicAdd(acc + r * s.CIg + a.idx, -(double)a.v);
                if (BOUND) {
                    const Route c = route_upper(pb[u], gb[u]);
                    if (c.idx < s.CIg) atomicAdd(acc + r * s.CIg + c.idx, -(double)c.v);
                }
            }
        }
    }
    __syncthreads();
    float* dst = gw + w_off(s, g, co0, 0);
    for (int i = threadIdx.x; i < nr * s.CIg; i += kGwWideThreads) {
        const float v = (float)acc[i];
        if (nsplit == 1) dst[i] = v;
        else if (v != 0.f) atomicAdd(dst + i, v);
    }
}

// grad_input as images [B, C, H, W]: one workgroup per (b, g, slab of CS image channels of the group).
// LDS: [BOUND ? 2 : 1][CS][H * W] gradient planes, then the window origin of every output position (two int16).
// Every workgroup walks over all codes of its sample, most of which name a channel outside its slab: those are
// dismissed with one comparison, and the loads of four codes are in flight at a time.
constexpr int kImageThreads = 1024;
template <bool BOUND>
__global__ __launch_bounds__(kImageThreads) void scatter_gx_image_kernel(
    const float* __restrict__ g1, const float* __restrict__ g2, const int32_t* __restrict__ p1,
    const int32_t* __restrict__ p2, float* __restrict__ gx1, float* __restrict__ gx2, const Geom s, const PatchMap pm,
    int CS, int nslab) {
    extern __shared__ float tile[];
    constexpr int NT = kImageThreads, UN = 4;
    unsigned id = blockIdx.x;
    const int slab = (int)(id % (unsigned)nslab);
    id /= (unsigned)nslab;
    const int g = (int)(id % (unsigned)s.G), b = (int)(id / (unsigned)s.G);
    const int c0 = slab * CS, cs = min(CS, pm.cg - c0);
    const int plane = pm.H * pm.W;
    const int ntile = (BOUND ? 2 : 1) * CS * plane;
    uint32_t* origin = reinterpret_cast<uint32_t*>(tile + ntile);
    for (int i = threadIdx.x; i < ntile; i += NT) tile[i] = 0.f;
    for (int hw = threadIdx.x; hw < s.HW; hw += NT) {
        int ih0, iw0;
        patch_origin(pm, hw, ih0, iw0);
        origin[hw] = ((uint32_t)ih0 << 16) | ((uint32_t)iw0 & 0xffffu);
    }
    __syncthreads();
    const unsigned k_lo = (unsigned)(c0 * pm.taps), k_n = (unsigned)(cs * pm.taps);  // the slab's range of k
    auto add = [&](const Route& r, long i) __attribute__((always_inline)) {
        // codes of other slabs, "no gradient" (target -1) and corrupt codes (idx beyond CIg) all end here
        const unsigned kk = (unsigned)r.idx - k_lo;
        if (r.target < 0 || kk >= k_n) return;
        const int hw = (int)(i % s.HW);
        const int cl = small_div((int)kk, pm.taps, pm.inv_taps), tap = (int)kk - cl * pm.taps;
        const int ti = small_div(tap, pm.kw, pm.inv_kw), tj = tap - ti * pm.kw;
        const uint32_t og = origin[hw];
        const int ih = (int)(int16_t)(og >> 16) + ti * pm.dh, iw = (int)(int16_t)(og & 0xffffu) + tj * pm.dw;
        if ((unsigned)ih >= (unsigned)pm.H || (unsigned)iw >= (unsigned)pm.W) return;  // the winner sits in the padding
        atomicAdd(tile + ((long)r.target * CS + cl) * plane + ih * pm.W + iw, r.v);
    };
    // element i of the sample's (co, hw) plane, hw fastest: adjacent lanes read adjacent codes
    const long obase = y_off(s, b, g, 0, 0);
    const long total = (long)s.COg * s.HW;
    for (long i0 = threadIdx.x; i0 < total; i0 += NT * UN) {
        int32_t c1[UN], c2[UN];
        float v1[UN], v2[UN];
#pragma unroll
        for (int u = 0; u < UN; u++) {
            const long i = i0 + u * NT;
            const bool ok = i < total;
            c1[u] = ok ? p1[obase + i] : (int32_t)kNoGradId;
            v1[u] = ok ? g1[obase + i] : 0.f;
            if (BOUND) {
                c2[u] = ok ? p2[obase + i] : (int32_t)kNoGradId;
                v2[u] = ok ? g2[obase + i] : 0.f;
            }
        }
#pragma unroll
        for (int u = 0; u < UN; u++) {
            const long i = i0 + u * NT;
            add(BOUND ? route_lower(c1[u], v1[u]) : route_inf(c1[u], v1[u]), i);
            if (BOUND) add(route_upper(c2[u], v2[u]), i);
        }
    }
    __syncthreads();
    const long base = (((long)b * pm.C + g * pm.cg + c0)) * plane;
    const int n = cs * plane;
    if (plane % 4 == 0 && (uintptr_t)gx1 % 16 == 0 && (!BOUND || (uintptr_t)gx2 % 16 == 0)) {
        for (int i = threadIdx.x; i < n / 4; i += NT) {
            reinterpret_cast<float4*>(gx1 + base)[i] = reinterpret_cast<const float4*>(tile)[i];
            if (BOUND) reinterpret_cast<float4*>(gx2 + base)[i] = reinterpret_cast<const float4*>(tile + CS * plane)[i];
        }
    } else {
        for (int i = threadIdx.x; i < n; i += NT) {
            gx1[base + i] = tile[i];
            if (BOUND) gx2[base + i] = tile[CS * plane + i];
        }
    }
}

// ---- images, by blocks of output rows -------------------------------------------------------------------
// A workgroup owns a few whole output rows of one sample (image_row_blocks) and every output channel of the group:
// the image rows under their windows, all channels, padding included, are a block of LDS in which every code of
// the workgroup's outputs is ONE float add (a per-k table entry plus a per-position offset) — no code is read by a
// workgroup that has no use for it, where the slab kernel below reads every code of a sample once per channel slab.
// Neighbouring row blocks share the image rows between their windows, so the block leaves through global float adds
// into a gradient cleared beforehand (cells that received nothing, and the padding, are not written).
template <bool BOUND>
__global__ __launch_bounds__(1024) void scatter_gx_rowblock_kernel(const float* __restrict__ g1, const float* __restrict__ g2,
                                                                  const int32_t* __restrict__ p1,
                                                                  const int32_t* __restrict__ p2, float* __restrict__ gx1,
                                                                  float* __restrict__ gx2, const Geom s, const PatchMap pm,
                                                                  const ImageRowBlocks rg) {
    extern __shared__ float lds[];
    constexpr int NX = BOUND ? 2 : 1;
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6), nwave = (int)blockDim.x >> 6, nthr = (int)blockDim.x;
    unsigned id = blockIdx.x;
    const int rb = (int)(id % (unsigned)rg.nrb);
    id /= (unsigned)rg.nrb;
    const int g = (int)(id % (unsigned)s.G), b = (int)(id / (unsigned)s.G);
    const int cg = pm.cg, E = rg.E, K = s.CIg, OW = pm.OW, OH = s.HW / pm.OW;
    const int K4 = (K + 3) & ~3;
    int* __restrict__ tab = reinterpret_cast<int*>(lds);  // [K4]: tap of k as an offset in the block
    float* __restrict__ acc = lds + K4;                    // [NX][cg][E]
    const int oh0 = rb * rg.R, nrow = min(rg.R, OH - oh0), npos = nrow * OW, hw0 = oh0 * OW;
    const int ih_base = oh0 * pm.sh - pm.ph;
    for (int k = tid; k < K; k += nthr) {
        const int cl = small_div(k, pm.taps, pm.inv_taps), tap = k - cl * pm.taps;
        const int ti = small_div(tap, pm.kw, pm.inv_kw), tj = tap - ti * pm.kw;
        tab[k] = cl * E + ti * pm.dh * rg.pitch + tj * pm.dw;
    }
    for (int i = tid; i < NX * cg * E; i += nthr) acc[i] = 0.f;
    __syncthreads();

    const int nmacro = (npos + 63) >> 6;  // blocks of 64 consecutive positions of one output channel
    const int total = s.COg * nmacro;
    constexpr int UN = 4;  // steps whose codes and gradients are requested together
#pragma unroll 1
    for (int it0 = wave; it0 < total; it0 += nwave * UN) {
        int32_t c1[UN], c2[UN];
        float v1[UN], v2[UN];
        int poff[UN];
#pragma unroll
        for (int u = 0; u < UN; u++) {
            const int it = it0 + u * nwave;
            const int n = it / nmacro, p = (it - n * nmacro) * 64 + lane;
            const bool live = it < total && p < npos;
            const long o = live ? y_off(s, b, g, n, hw0 + p) : 0;
            c1[u] = live ? p1[o] : (BOUND ? (int32_t)kNoGradId : 0);
            v1[u] = live ? g1[o] : 0.f;
            if (BOUND) {
                c2[u] = live ? p2[o] : 0;
                v2[u] = live ? g2[o] : 0.f;
            }
            const int pr = small_div(p, OW, rg.inv_ow), pc = p - pr * OW;
            poff[u] = live ? pr * pm.sh * rg.pitch + pc * pm.sw : -1;
        }
#pragma unroll
        for (int u = 0; u < UN; u++) {
            if (poff[u] < 0) continue;
            const Route a = BOUND ? route_lower(c1[u], v1[u]) : route_inf(c1[u], v1[u]);
            if (a.target >= 0 && a.idx < K && a.v != 0.f) atomicAdd(&acc[a.target * cg * E + tab[a.idx] + poff[u]], a.v);
            if (BOUND) {
                const Route c = route_upper(c2[u], v2[u]);
                if (c.idx < K && c.v != 0.f) atomicAdd(&acc[c.target * cg * E + tab[c.idx] + poff[u]], c.v);
            }
        }
    }
    __syncthreads();

    // ---- the block into the image gradient: a wave takes whole channels, as the staging of the second pass does
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
    const long img = ((long)b * pm.C + (long)g * cg) * plane;
    for (int c = wave; c < cg; c += nwave) {
#pragma unroll
        for (int q = 0; q < kRiMaxSlots; q++) {
            if (64 * q < E && ok[q]) {
                const float a = acc[c * E + lane + 64 * q];
                if (a != 0.f) atomicAdd(gx1 + img + c * plane + goff[q], a);
                if (BOUND) {
                    const float a2 = acc[(cg + c) * E + lane + 64 * q];
                    if (a2 != 0.f) atomicAdd(gx2 + img + c * plane + goff[q], a2);
                }
            }
        }
    }
}

// The same by blocks of IMAGE rows: a workgroup owns RI whole rows of every channel of one sample's group, reads the
// codes of all output rows whose windows touch them (the rows between two blocks are read by both: (RI + reach) / RI
// times the codes, reach = (kh - 1) dh rows), keeps the adds that land in its rows and writes them once, coalesced:
// no global atomics, no cleared gradient.  A tap is one table word (channel << 16 | dy << 8 | dx).
struct ImageRowOwners {
    int RI;    // image rows per workgroup
    int nib;   // row blocks per sample
    float inv_ow;
};
// ACC: float, or double where the rows still fit then (see "sums in double precision" above).
template <bool BOUND, typename ACC>
__global__ __launch_bounds__(1024) void scatter_gx_ownrows_kernel(const float* __restrict__ g1, const float* __restrict__ g2,
                                                                 const int32_t* __restrict__ p1,
                                                                 const int32_t* __restrict__ p2, float* __restrict__ gx1,
                                                                 float* __restrict__ gx2, const Geom s, const PatchMap pm,
                                                                 const ImageRowOwners ro) {
    extern __shared__ __align__(16) float lds[];
    constexpr int NX = BOUND ? 2 : 1;
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6), nwave = (int)blockDim.x >> 6, nthr = (int)blockDim.x;
    unsigned id = blockIdx.x;
    const int ib = (int)(id % (unsigned)ro.nib);
    id /= (unsigned)ro.nib;
    const int g = (int)(id % (unsigned)s.G), b = (int)(id / (unsigned)s.G);
    const int cg = pm.cg, K = s.CIg, OW = pm.OW, OH = s.HW / pm.OW, W = pm.W, RI = ro.RI;
    const int K4 = (K + 3) & ~3, kh = pm.taps / pm.kw;
    int* __restrict__ tab = reinterpret_cast<int*>(lds);  // [K4]
    ACC* __restrict__ acc = reinterpret_cast<ACC*>(lds + K4);  // [NX][cg][RI][W]  (K4 floats: 16-byte aligned)
    const int r0 = ib * RI, rows = min(RI, pm.H - r0), cell = RI * W;
    // output rows whose windows reach the rows [r0, r0 + rows)
    const int lo_num = r0 + pm.ph - (kh - 1) * pm.dh;
    const int oh_lo = lo_num <= 0 ? 0 : (lo_num + pm.sh - 1) / pm.sh;
    const int oh_hi = min(OH - 1, (r0 + rows - 1 + pm.ph) / pm.sh);
    const int npos = oh_hi >= oh_lo ? (oh_hi - oh_lo + 1) * OW : 0, hw0 = oh_lo * OW;
    for (int k = tid; k < K; k += nthr) tab[k] = pack_tap(patch_tap(pm, 0, k));
    for (int i = tid; i < NX * cg * cell; i += nthr) acc[i] = (ACC)0;
    __syncthreads();

    const int nmacro = (npos + 63) >> 6;
    const int total = s.COg * nmacro;
    constexpr int UN = 4;
    auto add = [&](const Route& a, int rowbase, int colbase) __attribute__((always_inline)) {
        if (a.target < 0 || a.idx >= K || a.v == 0.f) return;
        const PatchTap t = unpack_tap(tab[a.idx]);
        const int row = rowbase + t.dy, col = colbase + t.dx;
        if ((unsigned)row < (unsigned)rows && (unsigned)col < (unsigned)W)
            atomicAdd(&acc[(a.target * cg + t.ch) * cell + row * W + col], (ACC)a.v);
    };
#pragma unroll 1
    for (int it0 = wave; it0 < total; it0 += nwave * UN) {
        int32_t c1[UN], c2[UN];
        float v1[UN], v2[UN];
        int rowbase[UN], colbase[UN];
        bool live[UN];
#pragma unroll
        for (int u = 0; u < UN; u++) {
            const int it = it0 + u * nwave;
            const int n = it / nmacro, p = (it - n * nmacro) * 64 + lane;
            live[u] = it < total && p < npos;
            const long o = live[u] ? y_off(s, b, g, n, hw0 + p) : 0;
            c1[u] = live[u] ? p1[o] : (BOUND ? (int32_t)kNoGradId : 0);
            v1[u] = live[u] ? g1[o] : 0.f;
            if (BOUND) {
                c2[u] = live[u] ? p2[o] : 0;
                v2[u] = live[u] ? g2[o] : 0.f;
            }
            const int pr = small_div(p, OW, ro.inv_ow), pc = p - pr * OW;
            rowbase[u] = (oh_lo + pr) * pm.sh - pm.ph - r0;
            colbase[u] = pc * pm.sw - pm.pw;
        }
#pragma unroll
        for (int u = 0; u < UN; u++) {
            if (!live[u]) continue;
            add(BOUND ? route_lower(c1[u], v1[u]) : route_inf(c1[u], v1[u]), rowbase[u], colbase[u]);
            if (BOUND) add(route_upper(c2[u], v2[u]), rowbase[u], colbase[u]);
        }
    }
    __syncthreads();
    // ---- my rows of every channel: rows * W contiguous floats per channel
    const long plane = (long)pm.H * W;
    const long img = ((long)b * pm.C + (long)g * cg) * plane + (long)r0 * W;
    const int n = rows * W;
    const bool vec = n % 4 == 0 && cell % 4 == 0 && plane % 4 == 0 && (r0 * W) % 4 == 0 && (uintptr_t)gx1 % 16 == 0 &&
                     (!BOUND || (uintptr_t)gx2 % 16 == 0);
    auto sum4 = [&](int off) -> float4 {
        return make_float4((float)acc[off], (float)acc[off + 1], (float)acc[off + 2], (float)acc[off + 3]);
    };
    if (vec) {
        const int n4 = n / 4;
        for (int i = tid; i < cg * n4; i += nthr) {
            const int c = i / n4, e = (i - c * n4) * 4;
            *reinterpret_cast<float4*>(gx1 + img + c * plane + e) = sum4(c * cell + e);
            if (BOUND) *reinterpret_cast<float4*>(gx2 + img + c * plane + e) = sum4((cg + c) * cell + e);
        }
    } else {
        for (int i = tid; i < cg * n; i += nthr) {
            const int c = i / n, e = i - c * n;
            gx1[img + c * plane + e] = (float)acc[c * cell + e];
            if (BOUND) gx2[img + c * plane + e] = (float)acc[(cg + c) * cell + e];
        }
    }
}

// NORM_DIST_SCATTER_F64=0: float adds in LDS everywhere (tuning / test aid, read at every call)
static bool scatter_f64_enabled() {
    const char* e = getenv("NORM_DIST_SCATTER_F64");
    return e == nullptr || e[0] != '0';
}
constexpr int kScatterLdsBudget = 96 * 1024;
constexpr int kScatterTileBudget = 72 * 1024;  // two workgroups per CU

// Image-gradient path of the convolutional layer; returns -1 (nothing launched) when a plane of the image or a
// weight row does not fit the LDS budgets.
template <bool BOUND>
static int scatter_backward_images(const float* g1, const float* g2, const int32_t* p1, const int32_t* p2, const Geom& s,
                                   const PatchMap& pm, float* gx1, float* gx2, float* gw, hipStream_t st) {
    const int nx = BOUND ? 2 : 1;
    const long plane = (long)pm.H * pm.W;
    const long fixed = (long)s.HW * 4, per_ch = nx * plane * 4;
    if (gw && (size_t)s.CIg * sizeof(float) > (size_t)kScatterLdsBudget) return -1;
    // grad_weight launch parameters (shared by both grad_input routes)
    int R = 1, ncb = 0, nsplit = 1;
    const bool gw_wide = scatter_f64_enabled() && (size_t)s.CIg * sizeof(double) <= (size_t)kScatterLdsBudget;
    auto prepare_gw = [&]() -> int {
        NDIST_HIP_TRY(hipFuncSetAttribute(gw_wide ? reinterpret_cast<const void*>(&scatter_gw_split_f64_kernel<BOUND>)
                                                   : reinterpret_cast<const void*>(&scatter_gw_split_kernel<BOUND>),
                                          hipFuncAttributeMaxDynamicSharedMemorySize, kScatterLdsBudget));
        R = (int)((size_t)kScatterLdsBudget / ((size_t)s.CIg * (gw_wide ? sizeof(double) : sizeof(float))));
        R = R > 4 ? 4 : R;
        ncb = ceil_div(s.COg, R);
        nsplit = ceil_div((gw_wide ? 1 : 4) * device_info().num_cu, ncb * s.G);
        nsplit = nsplit > s.B ? s.B : nsplit;
        nsplit = nsplit > 65535 ? 65535 : nsplit;
        return nsplit > 1 ? fill_zero(gw, (long)s.COg * s.G * s.CIg, st) : 0;
    };
    auto launch_gw = [&]() -> int {
        if (gw_wide) {
            hipLaunchKernelGGL(scatter_gw_split_f64_kernel<BOUND>, dim3(ncb, s.G, nsplit), dim3(kGwWideThreads),
                               (size_t)R * s.CIg * sizeof(double), st, g1, g2, p1, p2, gw, s, R, nsplit);
        } else {
            hipLaunchKernelGGL(scatter_gw_split_kernel<BOUND>, dim3(ncb, s.G, nsplit), dim3(256),
                               (size_t)R * s.CIg * sizeof(float), st, g1, g2, p1, p2, gw, s, R, nsplit);
        }
        return hip_failed(hipGetLastError()) ? 4 : 0;
    };
    // Tuning / test aid: NORM_DIST_SCATTER_ROWBLOCKS=0 keeps the slab kernel, =1 the blocks of output rows.
    const char* sw = getenv("NORM_DIST_SCATTER_ROWBLOCKS");
    // By blocks of image rows, where a block can be at least twice as high as the windows reach (at most 1.5 times
    // the codes read) and a tap packs into a word: two workgroups per compute unit if that height fits half the LDS,
    // else one of 1024 threads.
    if ((sw == nullptr || (sw[0] != '0' && sw[0] != '1')) && pm.packable && s.CIg <= kRiMaxK && pm.OW > 0) {
        const int kh = pm.taps / pm.kw, reach = (kh - 1) * pm.dh;
        const size_t tabb = (size_t)((s.CIg + 3) & ~3) * sizeof(float);
        const int want = std::max(2 * reach, 1);
        // sums in doubles where a block of rows still fits then, else in floats
        bool wide = scatter_f64_enabled();
        size_t per_row = 0;
        int RI = 0, threads = 512;
        for (int attempt = 0; attempt < 2; attempt++) {
            per_row = (size_t)nx * pm.cg * pm.W * (wide ? sizeof(double) : sizeof(float));
            RI = (int)(((size_t)kRiLdsBudget / 2 - tabb) / per_row);
            threads = 512;
            if (RI < want) {
                RI = (int)(((size_t)kRiLdsBudget - tabb) / per_row);
                threads = 1024;
            }
            RI = std::min(RI, pm.H);
            if (!wide || RI >= (nx == 2 ? std::max(reach, 1) : want) || RI == pm.H) break;
            wide = false;
        }
        const long nwg = RI > 0 ? (long)s.B * s.G * ceil_div(pm.H, RI) : 0;
        if ((RI >= want || RI == pm.H || (wide && nx == 2 && RI >= std::max(reach, 1))) && RI > 0 && nwg < (1L << 31)) {
            const ImageRowOwners ro{RI, ceil_div(pm.H, RI), 1.0f / (float)pm.OW};
            const void* kern = wide ? reinterpret_cast<const void*>(&scatter_gx_ownrows_kernel<BOUND, double>)
                                    : reinterpret_cast<const void*>(&scatter_gx_ownrows_kernel<BOUND, float>);
            NDIST_HIP_TRY(hipFuncSetAttribute(kern, hipFuncAttributeMaxDynamicSharedMemorySize, kRiLdsBudget));
            if (gw) {
                if (int rc = prepare_gw()) return rc;
            }
            KernelTimer timer(st);  // both kernels together
            if (wide)
                hipLaunchKernelGGL((scatter_gx_ownrows_kernel<BOUND, double>), dim3((unsigned)nwg), dim3(threads),
                                   tabb + (size_t)RI * per_row, st, g1, g2, p1, p2, gx1, gx2, s, pm, ro);
            else
                hipLaunchKernelGGL((scatter_gx_ownrows_kernel<BOUND, float>), dim3((unsigned)nwg), dim3(threads),
                                   tabb + (size_t)RI * per_row, st, g1, g2, p1, p2, gx1, gx2, s, pm, ro);
            if (hip_failed(hipGetLastError())) return 4;
            return gw ? launch_gw() : 0;
        }
    }
    // by blocks of output rows where the rows under a block fit LDS
    {
        ImageRowBlocks rg{};
        size_t lds = 0;
        if ((sw == nullptr || sw[0] != '0') && image_row_blocks(s, pm, nx, &rg, &lds)) {
            NDIST_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void*>(&scatter_gx_rowblock_kernel<BOUND>),
                                              hipFuncAttributeMaxDynamicSharedMemorySize, kRiLdsBudget));
            if (gw) {
                if (int rc = prepare_gw()) return rc;
            }
            int rc = fill_zero(gx1, (long)s.B * pm.C * plane, st);
            if (!rc && BOUND) rc = fill_zero(gx2, (long)s.B * pm.C * plane, st);
            if (rc) return rc;
            KernelTimer timer(st);  // both kernels together
            const int threads = 2 * lds <= (size_t)kRiLdsBudget ? 512 : 1024;
            hipLaunchKernelGGL(scatter_gx_rowblock_kernel<BOUND>, dim3((unsigned)((long)s.B * s.G * rg.nrb)), dim3(threads),
                               lds, st, g1, g2, p1, p2, gx1, gx2, s, pm, rg);
            if (hip_failed(hipGetLastError())) return 4;
            return gw ? launch_gw() : 0;
        }
    }
    if (pm.ph >= 8192 || pm.pw >= 8192) return -1;  // window origins are packed into 16 bits (the plane bound limits H, W)
    if (fixed + per_ch > kScatterTileBudget) return -1;
    int CS = (int)((kScatterTileBudget - fixed) / per_ch);
    CS = CS > pm.cg ? pm.cg : CS;
    const int nslab = ceil_div(pm.cg, CS);
    const long nwg = (long)s.B * s.G * nslab;
    if (nslab > 16 || nwg >= (1L << 31)) return -1;
    NDIST_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void*>(&scatter_gx_image_kernel<BOUND>),
                                      hipFuncAttributeMaxDynamicSharedMemorySize, kScatterTileBudget));
    if (gw) {
        if (int rc = prepare_gw()) return rc;
    }
    KernelTimer timer(st);  // both kernels together
    hipLaunchKernelGGL(scatter_gx_image_kernel<BOUND>, dim3((unsigned)nwg), dim3(kImageThreads),
                       (size_t)(fixed + (long)CS * per_ch), st, g1, g2, p1, p2, gx1, gx2, s, pm, CS, nslab);
    if (hip_failed(hipGetLastError())) return 4;
    return gw ? launch_gw() : 0;
}

template <bool BOUND>
static int scatter_backward(const float* g1, const float* g2, const int32_t* p1, const int32_t* p2, const Geom& s,
                            float* gx1, float* gx2, float* gw, hipStream_t st) {
    const int nx = BOUND ? 2 : 1;
    const size_t gx_lds = (size_t)nx * s.CIg * sizeof(float);
    if (s.HW == 1 && gx_lds <= (size_t)kScatterLdsBudget) {
        const bool gx_wide = scatter_f64_enabled() && 2 * gx_lds <= (size_t)kScatterLdsBudget;
        NDIST_HIP_TRY(hipFuncSetAttribute(gx_wide ? reinterpret_cast<const void*>(&scatter_gx_rows_kernel<BOUND, double>)
                                                  : reinterpret_cast<const void*>(&scatter_gx_rows_kernel<BOUND, float>),
                                          hipFuncAttributeMaxDynamicSharedMemorySize, kScatterLdsBudget));
        NDIST_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void*>(&scatter_gw_rows_kernel<BOUND>),
                                          hipFuncAttributeMaxDynamicSharedMemorySize, kScatterLdsBudget));
        KernelTimer timer(st);  // both row kernels together
        // a row of 2048 outputs and more gets 1024 threads: the kernel has one workgroup per batch row and lives on
        // how many loads each of them keeps in flight
        const dim3 gx_grid(s.B, s.G), gx_block(s.COg >= 2048 ? 1024 : 256);
        if (gx_wide)
            hipLaunchKernelGGL((scatter_gx_rows_kernel<BOUND, double>), gx_grid, gx_block, 2 * gx_lds, st, g1, g2, p1, p2,
                               gx1, gx2, s);
        else
            hipLaunchKernelGGL((scatter_gx_rows_kernel<BOUND, float>), gx_grid, gx_block, gx_lds, st, g1, g2, p1, p2, gx1,
                               gx2, s);
        if (hip_failed(hipGetLastError())) return 4;
        if (gw) {
            int R = (int)((size_t)kScatterLdsBudget / ((size_t)s.CIg * sizeof(float)));
            // R >= 1 because one row fits the budget.  Two rows: with the XCD-aware numbering the L2 makes up for the
            // short segments, and four workgroups of 2 x 20 KB per compute unit overlap their fill, scatter and
            // store phases better than two of 4 x 20 KB (31.7 against 36.5 us at 512 x 5120 x 5120)
            R = R > 2 ? 2 : R;
            {   // tuning aid: NORM_DIST_GW_ROWS=<n> rows of grad_weight per workgroup
                static const char* force = getenv("NORM_DIST_GW_ROWS");
                if (force != nullptr && atoi(force) >= 1) R = atoi(force) < R ? atoi(force) : R;
            }
            hipLaunchKernelGGL(scatter_gw_rows_kernel<BOUND>, dim3(ceil_div(s.COg, R), s.G), dim3(256),
                               (size_t)R * s.CIg * sizeof(float), st, g1, g2, p1, p2, gw, s, R);
            if (hip_failed(hipGetLastError())) return 4;
        }
        return 0;
    }
    if (s.HW > 1 && (size_t)s.CIg * sizeof(float) <= (size_t)kScatterLdsBudget) {
        // grad_input tiles: the largest ci slab that fits; give up when the codes would be re-read too often
        const int cs_max = kScatterTileBudget / (nx * kScatterHB * (int)sizeof(float));
        const int CS = s.CIg < cs_max ? s.CIg : cs_max;
        const int nslab = ceil_div(s.CIg, CS), nhb = ceil_div(s.HW, kScatterHB);
        const long nwg = (long)s.B * s.G * nhb * nslab;
        if (nslab <= 8 && nwg < (1L << 31)) {
            NDIST_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void*>(&scatter_gx_tile_kernel<BOUND>),
                                              hipFuncAttributeMaxDynamicSharedMemorySize, kScatterTileBudget));
            // (sums in doubles where a row of them fits: see scatter_gw_split_f64_kernel)
            const bool gw_wide = scatter_f64_enabled() && (size_t)s.CIg * sizeof(double) <= (size_t)kScatterLdsBudget;
            NDIST_HIP_TRY(hipFuncSetAttribute(gw_wide ? reinterpret_cast<const void*>(&scatter_gw_split_f64_kernel<BOUND>)
                                                       : reinterpret_cast<const void*>(&scatter_gw_split_kernel<BOUND>),
                                              hipFuncAttributeMaxDynamicSharedMemorySize, kScatterLdsBudget));
            int R = (int)((size_t)kScatterLdsBudget / ((size_t)s.CIg * (gw_wide ? sizeof(double) : sizeof(float))));
            R = R > 4 ? 4 : R;
            const int ncb = ceil_div(s.COg, R);
            // enough workgroups to cover the device about four times (once with the 1024-thread workgroups of the
            // kernel that sums in doubles), at most one share per sample
            int nsplit = ceil_div((gw_wide ? 1 : 4) * device_info().num_cu, ncb * s.G);
            nsplit = nsplit > s.B ? s.B : nsplit;
            nsplit = nsplit > 65535 ? 65535 : nsplit;
            if (gw && nsplit > 1) {
                const int rc = fill_zero(gw, (long)s.COg * s.G * s.CIg, st);
                if (rc) return rc;
            }
            KernelTimer timer(st);  // both tile kernels together
            hipLaunchKernelGGL(scatter_gx_tile_kernel<BOUND>, dim3((unsigned)nwg), dim3(256),
                               (size_t)nx * CS * kScatterHB * sizeof(float), st, g1, g2, p1, p2, gx1, gx2, s, CS, nslab,
                               nhb);
            if (hip_failed(hipGetLastError())) return 4;
            if (gw && gw_wide) {
                hipLaunchKernelGGL(scatter_gw_split_f64_kernel<BOUND>, dim3(ncb, s.G, nsplit), dim3(kGwWideThreads),
                                   (size_t)R * s.CIg * sizeof(double), st, g1, g2, p1, p2, gw, s, R, nsplit);
                if (hip_failed(hipGetLastError())) return 4;
            } else if (gw) {
                hipLaunchKernelGGL(scatter_gw_split_kernel<BOUND>, dim3(ncb, s.G, nsplit), dim3(256),
                                   (size_t)R * s.CIg * sizeof(float), st, g1, g2, p1, p2, gw, s, R, nsplit);
                if (hip_failed(hipGetLastError())) return 4;
            }
            return 0;
        }
    }
    int rc = fill_zero(gx1, (long)s.M * s.CIg * s.G, st);
    if (!rc && BOUND) rc = fill_zero(gx2, (long)s.M * s.CIg * s.G, st);
    if (!rc && gw) rc = fill_zero(gw, (long)s.COg * s.G * s.CIg, st);
    if (rc) return rc;
    const long total = (long)s.M * s.COg * s.G;
    hipLaunchKernelGGL(scatter_atomic_kernel<BOUND>, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, st, g1, g2, p1,
                       p2, gx1, gx2, gw, s, total);
    return hip_failed(hipGetLastError()) ? 4 : 0;
}

int launch_inf_backward(const float* gout, const int32_t* pos, const Geom& s, float* gx, float* gw, hipStream_t st,
                        const UnfoldGeom* cv) {
    if (cv != nullptr)
        return scatter_backward_images<false>(gout, nullptr, pos, nullptr, s, make_patch_map(*cv, s.G), gx, nullptr, gw, st);
    return scatter_backward<false>(gout, nullptr, pos, nullptr, s, gx, nullptr, gw, st);
}

int launch_bound_backward(const float* gl, const float* gu, const int32_t* pl, const int32_t* pu, const Geom& s,
                          float* gxl, float* gxu, float* gw, hipStream_t st, const UnfoldGeom* cv) {
    if (cv != nullptr)
        return scatter_backward_images<true>(gl, gu, pl, pu, s, make_patch_map(*cv, s.G), gxl, gxu, gw, st);
    return scatter_backward<true>(gl, gu, pl, pu, s, gxl, gxu, gw, st);
}

}  // namespace ndist
