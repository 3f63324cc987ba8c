// Forward kernel for problems with few outputs and a long reduction (the 10-class last layer of the MLP:
// 512 x 10 outputs over 5120 inputs).  The tiled kernel would cover such a problem with a handful of workgroups that
// each walk the whole k range alone; here the k range is spread over the 64 lanes of a wave instead: one wave owns
// 2 rows x 4 co, every lane takes 4 consecutive k of each 256-wide step (one 16-byte load per operand row, 1 KiB
// contiguous per wave), accumulates with the same operator policies as the tiled kernel, and the lanes are merged
// with a butterfly of cross-lane shuffles at the end.  The four waves of a workgroup share one such block of outputs
// and take every fourth step each (a wave alone would walk K / 256 dependent memory latencies: 37 us for the 512 x 10
// layer); their results meet in LDS after the one barrier of the kernel.  Fully-connected layout only.
//
// Arg-max bookkeeping: a lane's "tile" is its 4 consecutive k of one step (tile index step * 64 + lane, so tiles
// are ordered like their k); the rescan kernels then run with a tile length of 4.
// (This file is a part of fwd_tile.h, which includes it between the tiled kernel and the launcher.)
#pragma once

namespace ndist {

constexpr int kSkinnyRows = 2, kSkinnyCols = 4, kSkinnyKT = 4;
constexpr long kSkinnyMaxOutputs = 32768;  // above this the operand traffic through L2 outweighs the parallelism
constexpr int kSkinnyMinK = 256;

template <class Acc>
__device__ __forceinline__ Acc shuffle_xor_acc(const Acc& a, int mask) {
    constexpr int NF = sizeof(Acc) / 4;
    int f[NF];
    __builtin_memcpy(f, &a, sizeof(Acc));
#pragma unroll
    for (int q = 0; q < NF; q++) f[q] = __shfl_xor(f[q], mask, 64);
    Acc r;
    __builtin_memcpy(&r, f, sizeof(Acc));
    return r;
}

template <class Op>
__global__ __launch_bounds__(256) void fwd_skinny_kernel(const FwdParams P, int nrp, int ncq) {
    constexpr int R = kSkinnyRows, TN = kSkinnyCols, NX = Op::NX;
    using Acc = typename Op::Acc;
    if (gate_closed(P)) return;
    const Geom& s = P.s;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    long wid = blockIdx.x;  // one block of outputs per workgroup: nobody leaves before the barrier
    const int cq = (int)(wid % ncq);
    wid /= ncq;
    const int rp = (int)(wid % nrp), g = (int)(wid / nrp);
    const int m0 = rp * R, n0 = cq * TN, K = s.CIg;

    Acc acc[R][TN];
#pragma unroll
    for (int r = 0; r < R; r++)
#pragma unroll
        for (int j = 0; j < TN; j++) Op::init(acc[r][j], P, (lane | wave) == 0 ? 0 : 1, m0 + r, n0 + j, g);

    const float* xrow[NX][R];
    const float* wrow[TN];
    bool xok[R], wok[TN];
#pragma unroll
    for (int r = 0; r < R; r++) {
        xok[r] = m0 + r < s.M;
        const long off = x_off(s, xok[r] ? m0 + r : 0, g, 0, 0);
        xrow[0][r] = P.x + off;
        if (NX == 2) xrow[NX - 1][r] = P.x2 + off;
    }
#pragma unroll
    for (int j = 0; j < TN; j++) {
        wok[j] = n0 + j < s.COg;
        wrow[j] = P.w + w_off(s, g, wok[j] ? n0 + j : 0, 0);
    }

    float4 xq[2][NX][R], wq[2][TN];
    auto fetch = [&](int slot, int k) {
#pragma unroll
        for (int a = 0; a < NX; a++)
#pragma unroll
            for (int r = 0; r < R; r++) xq[slot][a][r] = load4_guarded(xrow[a][r], k, K, xok[r], P.x_vec);
#pragma unroll
        for (int j = 0; j < TN; j++) wq[slot][j] = load4_guarded(wrow[j], k, K, wok[j], P.w_vec);
    };
    auto compute = [&](int slot, int tile) {
        if (NX == 2) {
            // an inverted box collapses to its midpoint (reference: core/cuda/bound_inf_dist_cuda.cu:63)
#pragma unroll
            for (int r = 0; r < R; r++) {
                float* a = reinterpret_cast<float*>(&xq[slot][0][r]);
                float* c = reinterpret_cast<float*>(&xq[slot][NX - 1][r]);
#pragma unroll
                for (int q = 0; q < 4; q++)
                    if (a[q] > c[q]) a[q] = c[q] = (a[q] + c[q]) * 0.5f;
            }
        }
        float w0[TN], w1[TN], w2[TN], w3[TN];
#pragma unroll
        for (int j = 0; j < TN; j++) { w0[j] = wq[slot][j].x; w1[j] = wq[slot][j].y; w2[j] = wq[slot][j].z; w3[j] = wq[slot][j].w; }
#pragma unroll
        for (int ph = 0; ph < Op::PHASES; ph++) {
#pragma unroll
            for (int r = 0; r < R; r++) {
                const float4 a = xq[slot][0][r];
                const float4 c = NX == 2 ? xq[slot][NX - 1][r] : make_float4(0.f, 0.f, 0.f, 0.f);
                Op::template row2<TN>(acc[r], P, ph, a.x, c.x, w0, a.y, c.y, w1);
                Op::template row2<TN>(acc[r], P, ph, a.z, c.z, w2, a.w, c.w, w3);
            }
#pragma unroll
            for (int r = 0; r < R; r++)
#pragma unroll
                for (int j = 0; j < TN; j++) Op::phase_end(acc[r][j], P, ph, tile);
        }
    };

    // my steps: wave, wave + 4, ... (the workgroup reads 4 KiB of every operand row at a time)
    const int nsteps = ceil_div(K, 256);
    if (wave < nsteps) fetch(0, wave * 256 + lane * 4);
    for (int it = wave; it < nsteps; it += 8) {
        if (it + 4 < nsteps) fetch(1, (it + 4) * 256 + lane * 4);
        compute(0, it * 64 + lane);
        if (it + 4 < nsteps) {
            if (it + 8 < nsteps) fetch(0, (it + 8) * 256 + lane * 4);
            compute(1, (it + 4) * 64 + lane);
        }
    }

    // ---- merge the lanes: after the butterfly every lane holds the result
#pragma unroll
    for (int mask = 32; mask >= 1; mask >>= 1)
#pragma unroll
        for (int r = 0; r < R; r++)
#pragma unroll
            for (int j = 0; j < TN; j++) {
                const Acc other = shuffle_xor_acc(acc[r][j], mask);
                Op::merge(acc[r][j], other, P);
            }

    // ---- merge the waves
    __shared__ Acc part[3][R][TN];
    if (wave != 0 && lane == 0) {
#pragma unroll
        for (int r = 0; r < R; r++)
#pragma unroll
            for (int j = 0; j < TN; j++) part[wave - 1][r][j] = acc[r][j];
    }
    __syncthreads();
    if (wave != 0) return;
#pragma unroll
    for (int q = 0; q < 3; q++)
#pragma unroll
        for (int r = 0; r < R; r++)
#pragma unroll
            for (int j = 0; j < TN; j++) {
                const Acc other = part[q][r][j];
                Op::merge(acc[r][j], other, P);
            }

    if (lane < R * TN) {
        constexpr int NOF = Op::NOF, NOI = Op::NOI;
        float* fo[2] = {P.out, P.out2};
        int32_t* io[2] = {P.pos, P.pos2};
#pragma unroll
        for (int r = 0; r < R; r++)
#pragma unroll
            for (int j = 0; j < TN; j++) {
                if (lane != r * TN + j) continue;
                if (m0 + r >= s.M || n0 + j >= s.COg) continue;
                float fv[NOF > 0 ? NOF : 1];
                int iv[NOI > 0 ? NOI : 1];
                Op::finalize(acc[r][j], P, fv, iv);
                const long o = y_off(s, m0 + r, g, n0 + j, 0);
#pragma unroll
                for (int q = 0; q < NOF; q++) fo[q][o] = fv[q];
#pragma unroll
                for (int q = 0; q < NOI; q++) io[q][o] = iv[q];
            }
    }
}

inline bool skinny_applies(const Geom& s) {
    return s.HW == 1 && s.CIg >= kSkinnyMinK && (long)s.M * s.COg * s.G <= kSkinnyMaxOutputs &&
           (long)ceil_div(s.CIg, kSkinnyKT) < (1L << 30);
}

template <class Op>
int launch_skinny(FwdParams P, hipStream_t st, int* chosen_kt) {
    const Geom& s = P.s;
    P.x_vec = s.CIg % 4 == 0 && (uintptr_t)P.x % 16 == 0 && (P.x2 == nullptr || (uintptr_t)P.x2 % 16 == 0);
    P.w_vec = s.CIg % 4 == 0 && (uintptr_t)P.w % 16 == 0;
    P.kt = kSkinnyKT;
    P.ksplit = 1;
    if (chosen_kt) *chosen_kt = P.kt;
    const int nrp = ceil_div(s.M, kSkinnyRows), ncq = ceil_div(s.COg, kSkinnyCols);
    const long nw = (long)s.G * nrp * ncq;
    KernelTimer timer(st);
    hipLaunchKernelGGL((fwd_skinny_kernel<Op>), dim3((unsigned)nw), dim3(256), 0, st, P, nrp, ncq);
    return hip_failed(hipGetLastError()) ? 4 : 0;
}

}  // namespace ndist
