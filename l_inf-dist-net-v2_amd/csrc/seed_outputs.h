// Seeds of the outputs for the operators that skip k-tiles: per output the larger of the two pairs at the k where its
// row of x, and where its row of w, is largest.  The work of one workgroup (64 rows x 64 columns of one group) as
// device functions: a kernel of their own runs them, and so does the hot-tile kernel in the launches in which the
// plan has decided against it (one launch less on the path where the dense kernels are gated off).
#pragma once

#include "ndist_common.h"

namespace ndist {

struct OutputSeedJob {
    const float* seed_x;  // per row of x: element of largest magnitude (the interval variant reads the box itself)
    const int32_t* seed_k;
    const float* seed_w;
    const int32_t* seed_wk;
    float* seed;   // interval bounds: seed of the upper reduction
    float* seed2;  // interval bounds: seed of the lower reduction
    int nmb, nnb;  // blocks of 64 rows / 64 columns
};
constexpr int kSeedTileFloats = 64 * 65;

// The pairs from the x seeds are gathered with the lanes along the rows (a wave then reads inside one row of w), the
// pairs from the w seeds with the lanes along the columns (inside one row of x), an LDS tile turns the first set
// around, and the seeds are written with the lanes along the columns.  lds: kSeedTileFloats floats.
__device__ __forceinline__ void norm_seed_outputs_block(const float* __restrict__ x, const float* __restrict__ w,
                                                        const Geom& s, const OutputSeedJob& job, unsigned id,
                                                        float* __restrict__ lds) {
    const int nb = (int)(id % (unsigned)job.nnb);
    id /= (unsigned)job.nnb;
    const int mb = (int)(id % (unsigned)job.nmb), g = (int)(id / (unsigned)job.nmb);
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int m0 = mb * 64, n0 = nb * 64;
    {
        const int m = m0 + lane;
        float sx = 0.f;
        int kx = 0;
        if (m < s.M) {
            sx = job.seed_x[(long)m * s.G + g];
            kx = job.seed_k[(long)m * s.G + g];
        }
#pragma unroll 4
        for (int c = wave * 16; c < wave * 16 + 16; c++) {
            const int n = n0 + c;
            float v = 0.f;
            if (m < s.M && n < s.COg) v = fabsf(sx - w[w_off(s, g, n, kx)]);
            lds[lane * 65 + c] = v;
        }
    }
    __syncthreads();
    {
        const int n = n0 + lane;
        float sw = 0.f;
        int kw = 0;
        if (n < s.COg) {
            sw = job.seed_w[g * s.COg + n];
            kw = job.seed_wk[g * s.COg + n];
        }
#pragma unroll 4
        for (int rr = wave * 16; rr < wave * 16 + 16; rr++) {
            const int m = m0 + rr;
            if (m < s.M && n < s.COg) {
                const int b = m / s.HW, hw = m - b * s.HW;
                const float v = fabsf(x[x_off(s, b, g, kw, hw)] - sw);
                job.seed[y_off(s, b, g, n, hw)] = fmaxf(fmaxf(lds[rr * 65 + lane], v), kEps);
            }
        }
    }
}

// The same for the interval bounds: seeds of the upper reduction (max of w - xL, xU - w) and of the lower one (min of
// the same two) at the k of the row seeds.  lds: 2 * kSeedTileFloats floats.
__device__ __forceinline__ void bound_seed_outputs_block(const float* __restrict__ xl, const float* __restrict__ xu,
                                                         const float* __restrict__ w, const Geom& s,
                                                         const OutputSeedJob& job, unsigned id, float* __restrict__ lds) {
    float* __restrict__ thi = lds;
    float* __restrict__ tlo = lds + kSeedTileFloats;
    const int nb = (int)(id % (unsigned)job.nnb);
    id /= (unsigned)job.nnb;
    const int mb = (int)(id % (unsigned)job.nmb), g = (int)(id / (unsigned)job.nmb);
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int m0 = mb * 64, n0 = nb * 64;
    {
        const int m = m0 + lane;
        float sl = 0.f, su = 0.f;
        int kx = 0;
        if (m < s.M) {
            kx = job.seed_k[(long)m * s.G + g];
            sl = xl[x_off(s, m, g, kx, 0)];
            su = xu[x_off(s, m, g, kx, 0)];
            if (sl > su) sl = su = (sl + su) * 0.5f;  // an inverted box collapses to its midpoint, as in the operator
        }
#pragma unroll 4
        for (int c = wave * 16; c < wave * 16 + 16; c++) {
            const int n = n0 + c;
            float hi = kEps, lo = -kEps;
            if (m < s.M && n < s.COg) {
                const float wv = w[w_off(s, g, n, kx)];
                const float t1 = wv - sl, t2 = su - wv;
                hi = fmaxf(t1, t2);
                lo = fminf(t1, t2);
            }
            thi[lane * 65 + c] = hi;
            tlo[lane * 65 + c] = lo;
        }
    }
    __syncthreads();
    {
        const int n = n0 + lane;
        float sw = 0.f;
        int kw = 0;
        if (n < s.COg) {
            sw = job.seed_w[g * s.COg + n];
            kw = job.seed_wk[g * s.COg + n];
        }
#pragma unroll 4
        for (int rr = wave * 16; rr < wave * 16 + 16; rr++) {
            const int m = m0 + rr;
            if (m < s.M && n < s.COg) {
                float vl = xl[x_off(s, m, g, kw, 0)], vu = xu[x_off(s, m, g, kw, 0)];
                if (vl > vu) vl = vu = (vl + vu) * 0.5f;
                const float t1 = sw - vl, t2 = vu - sw;
                job.seed[y_off(s, m, g, n, 0)] = fmaxf(fmaxf(fmaxf(t1, t2), thi[rr * 65 + lane]), kEps);
                job.seed2[y_off(s, m, g, n, 0)] = fminf(fminf(fminf(t1, t2), tlo[rr * 65 + lane]), -kEps);
            }
        }
    }
}

inline OutputSeedJob output_seed_job(const Geom& s, const SeedBuffers& sb) {
    return OutputSeedJob{sb.seed_x, sb.seed_k, sb.seed_w, sb.seed_wk, sb.seed, sb.seed2, ceil_div(s.M, 64), ceil_div(s.COg, 64)};
}

}  // namespace ndist
