// Issue-rate micro-benchmark of the gfx950 vector ALU for the instruction mixes of the distance kernels.
//
// Every mix is written in stages over CH independent chains (stage s of all chains, then stage s+1, ...), so that a
// wave has CH independent instructions between two dependent ones; the sweep is over CH = 1, 2, 4, 8 and over
// 1..8 waves per SIMD (256-thread workgroups, one wave per SIMD each, their number per compute unit pinned by the
// dynamic LDS size).  No memory traffic inside the timed loop (except the mix that reads LDS on purpose).
//
// Printed per case: SIMD cycles per wave64 instruction at the 2.4 GHz datasheet clock (wall time * 2.4e9 * SIMDs /
// wave instructions), the clock the part actually ran at during the case (s_memtime is the shader clock when it
// differs from the constant-rate s_memrealtime; otherwise 0 is printed and the clock has to come from counters:
// rocprofv3 --pmc GRBM_GUI_ACTIVE --kernel-trace), and cycles per pair for the mixes that model a kernel.
//   build:  make -C l_inf-dist-net-v2_amd/csrc microbench
//   run:    l_inf-dist-net-v2_amd/csrc/build/valu_issue [mix ... | n]
#include <hip/hip_runtime.h>

#include <cstdio>
#include <cstdlib>

#define CHECK(x)                                                           \
    do {                                                                   \
        hipError_t e_ = (x);                                               \
        if (e_ != hipSuccess) {                                            \
            printf("HIP error %d (%s) at line %d\n", (int)e_, hipGetErrorString(e_), __LINE__); \
            exit(1);                                                       \
        }                                                                  \
    } while (0)

enum Mix {
    FMA3 = 0,     // acc = fma(a, b, acc), three different registers
    MUL,          // acc = acc * a
    ADD,          // acc = acc + a
    MUL_S,        // acc = s * acc          (scalar operand)
    FMA_S,        // acc = fma(s, a, acc)   (scalar operand)
    MAX,          // acc = max(acc, a)
    MAX3,         // acc = max3(acc, |a|, |b|)
    MOV_S,        // v = s
    ADD_DPP,      // acc = acc + quad_perm(a)
    EXP,          // acc = exp2(acc)
    P8_FWD,       // d = x - w ; d = d*d ; d = d*d ; acc = fma(d, d, acc)                     1 pair
    P8_BWD,       // t = x - w ; v = s*t ; v2 = v*v ; v3 = v2*v ; v6 = v3*v3 ; gx += v*v6 ; gw += v*v6   1 term
    P8_BWD_V,     // the same with the factor in a vector register
    P8_BWD_LDS,   // P8_BWD_V plus one uniform-address ds_read_b128 per four terms (factors broadcast from LDS)
    INF,          // d0 = x - w0 ; d1 = x - w1 ; acc = max3(acc, |d0|, |d1|)                2 pairs
    BOUND,        // t1 = w - xl ; t2 = xu - w ; lo = min3(lo, t1, t2) ; hi = max3(hi, t1, t2)   1 pair
    GENP,         // d = x - w ; e = log2|d| ; e = p*e - c ; e = exp2(e) ; acc += e           1 pair
    GENP_BWD,     // t = x - w ; v = s*t ; e = log2|v| ; e = s*e ; e = exp2(e) ; gx += v*e ; gw += v*e   1 term
    NMIX
};

struct MixInfo {
    const char* name;
    int instr;     // vector instructions per chain and step
    double pairs;  // pairs (terms) per chain and step, 0 when the mix models no kernel
};
static const MixInfo kMix[NMIX] = {
    {"fma v,v,v", 1, 0},
    {"mul v,v", 1, 0},
    {"add v,v", 1, 0},
    {"mul s,v (scalar operand)", 1, 0},
    {"fma s,v,v (scalar operand)", 1, 0},
    {"max v,v", 1, 0},
    {"max3 v,|v|,|v|", 1, 0},
    {"mov v,s", 1, 0},
    {"add v,v quad_perm (DPP)", 1, 0},
    {"exp", 1, 0},
    {"p=8 forward: sub mul mul fma", 4, 1},
    {"p=8 backward: sub mul_s 3mul 2fma", 7, 1},
    {"p=8 backward, factor in a VGPR", 7, 1},
    {"p=8 backward, factors by ds_read_b128 broadcast", 7, 1},
    {"inf: sub sub max3 (2 pairs)", 3, 2},
    {"bounds: sub sub min3 max3", 4, 1},
    {"general p: sub log fma exp add", 5, 1},
    {"general p backward: sub mul_s log mul_s exp 2fma", 7, 1},
};

typedef float f4 __attribute__((ext_vector_type(4)));

// one step of MIX over CH chains, staged
template <int MIX, int CH, int NOPS>
__device__ __forceinline__ void step(float (&acc)[CH], float (&acc2)[CH], const float (&a)[CH], const float (&b)[CH], float sc,
                                     const float* lds) {
    float d[CH], e[CH], f[CH];
#define STAGE(...)                                                    \
    _Pragma("unroll") for (int c = 0; c < CH; c++) {                  \
        asm volatile(__VA_ARGS__);                                    \
        if constexpr (NOPS == 1) asm volatile("s_nop 0");             \
        if constexpr (NOPS == 2) asm volatile("s_nop 1");             \
        if constexpr (NOPS == 3) asm volatile("s_nop 2");             \
        if constexpr (NOPS == 4) asm volatile("s_nop 3");             \
    }
    if constexpr (MIX == FMA3) { STAGE("v_fma_f32 %0, %1, %2, %0" : "+v"(acc[c]) : "v"(a[c]), "v"(b[c])) }
    if constexpr (MIX == MUL) { STAGE("v_mul_f32 %0, %0, %1" : "+v"(acc[c]) : "v"(a[c])) }
    if constexpr (MIX == ADD) { STAGE("v_add_f32 %0, %0, %1" : "+v"(acc[c]) : "v"(a[c])) }
    if constexpr (MIX == MUL_S) { STAGE("v_mul_f32 %0, %1, %0" : "+v"(acc[c]) : "s"(sc)) }
    if constexpr (MIX == FMA_S) { STAGE("v_fma_f32 %0, %1, %2, %0" : "+v"(acc[c]) : "s"(sc), "v"(a[c])) }
    if constexpr (MIX == MAX) { STAGE("v_max_f32 %0, %0, %1" : "+v"(acc[c]) : "v"(a[c])) }
    if constexpr (MIX == MAX3) { STAGE("v_max3_f32 %0, %0, |%1|, |%2|" : "+v"(acc[c]) : "v"(a[c]), "v"(b[c])) }
    if constexpr (MIX == MOV_S) { STAGE("v_mov_b32 %0, %1" : "=v"(acc[c]) : "s"(sc)) }
    if constexpr (MIX == ADD_DPP) {
        STAGE("v_add_f32_dpp %0, %1, %0 quad_perm:[1,0,3,2] row_mask:0xf bank_mask:0xf" : "+v"(acc[c]) : "v"(a[c]))
    }
    if constexpr (MIX == EXP) { STAGE("v_exp_f32 %0, %0" : "+v"(acc[c])) }
    if constexpr (MIX == P8_FWD) {
        STAGE("v_sub_f32 %0, %1, %2" : "=v"(d[c]) : "v"(a[c]), "v"(b[c]))
        STAGE("v_mul_f32 %0, %0, %0" : "+v"(d[c]))
        STAGE("v_mul_f32 %0, %0, %0" : "+v"(d[c]))
        STAGE("v_fma_f32 %0, %1, %1, %0" : "+v"(acc[c]) : "v"(d[c]))
    }
    if constexpr (MIX == P8_BWD || MIX == P8_BWD_V || MIX == P8_BWD_LDS) {
        if constexpr (MIX == P8_BWD_LDS) {
            // factors of four terms per uniform-address 16-byte LDS read (the values are not used: the timing is)
#pragma unroll
            for (int c = 0; c < CH; c += 4) {
                f4 q;
                asm volatile("ds_read_b128 %0, %1" : "=v"(q) : "v"((unsigned)(size_t)lds + 16u * c));
                asm volatile("" ::"v"(q));
            }
        }
        STAGE("v_sub_f32 %0, %1, %2" : "=v"(d[c]) : "v"(a[c]), "v"(b[0]))
        if constexpr (MIX == P8_BWD) { STAGE("v_mul_f32 %0, %1, %0" : "+v"(d[c]) : "s"(sc)) }
        else { STAGE("v_mul_f32 %0, %1, %0" : "+v"(d[c]) : "v"(b[c])) }
        STAGE("v_mul_f32 %0, %1, %1" : "=v"(e[c]) : "v"(d[c]))
        STAGE("v_mul_f32 %0, %0, %1" : "+v"(e[c]) : "v"(d[c]))
        STAGE("v_mul_f32 %0, %0, %0" : "+v"(e[c]))
        STAGE("v_fma_f32 %0, %1, %2, %0" : "+v"(acc[c]) : "v"(d[c]), "v"(e[c]))
        STAGE("v_fma_f32 %0, %1, %2, %0" : "+v"(acc2[c]) : "v"(d[c]), "v"(e[c]))
        if constexpr (MIX == P8_BWD_LDS) asm volatile("s_waitcnt lgkmcnt(0)");
    }
    if constexpr (MIX == INF) {
        STAGE("v_sub_f32 %0, %1, %2" : "=v"(d[c]) : "v"(a[c]), "v"(b[c]))
        STAGE("v_sub_f32 %0, %2, %1" : "=v"(e[c]) : "v"(a[c]), "v"(b[c]))
        STAGE("v_max3_f32 %0, %0, |%1|, |%2|" : "+v"(acc[c]) : "v"(d[c]), "v"(e[c]))
    }
    if constexpr (MIX == BOUND) {
        STAGE("v_sub_f32 %0, %1, %2" : "=v"(d[c]) : "v"(a[c]), "v"(b[c]))
        STAGE("v_sub_f32 %0, %2, %1" : "=v"(e[c]) : "v"(a[c]), "v"(b[c]))
        STAGE("v_min3_f32 %0, %0, %1, %2" : "+v"(acc[c]) : "v"(d[c]), "v"(e[c]))
        STAGE("v_max3_f32 %0, %0, %1, %2" : "+v"(acc2[c]) : "v"(d[c]), "v"(e[c]))
    }
    if constexpr (MIX == GENP) {
        STAGE("v_sub_f32 %0, %1, %2" : "=v"(d[c]) : "v"(a[c]), "v"(b[c]))
        STAGE("v_log_f32 %0, |%0|" : "+v"(d[c]))
        STAGE("v_fma_f32 %0, %1, %0, %2" : "+v"(d[c]) : "v"(b[0]), "v"(a[c]))
        STAGE("v_exp_f32 %0, %0" : "+v"(d[c]))
        STAGE("v_add_f32 %0, %0, %1" : "+v"(acc[c]) : "v"(d[c]))
    }
    if constexpr (MIX == GENP_BWD) {
        STAGE("v_sub_f32 %0, %1, %2" : "=v"(d[c]) : "v"(a[c]), "v"(b[c]))
        STAGE("v_mul_f32 %0, %1, %0" : "+v"(d[c]) : "s"(sc))
        STAGE("v_log_f32 %0, |%1|" : "=v"(e[c]) : "v"(d[c]))
        STAGE("v_mul_f32 %0, %1, %0" : "+v"(e[c]) : "s"(sc))
        STAGE("v_exp_f32 %0, %0" : "+v"(e[c]))
        STAGE("v_fma_f32 %0, %1, %2, %0" : "+v"(acc[c]) : "v"(d[c]), "v"(e[c]))
        STAGE("v_fma_f32 %0, %1, %2, %0" : "+v"(acc2[c]) : "v"(d[c]), "v"(e[c]))
    }
#undef STAGE
    (void)f;
}

template <int MIX, int CH, int UNROLL, int NOPS>
__global__ __launch_bounds__(256) void mix_kernel(float* out, const float* in, int iters, float sc,
                                                  unsigned long long* clk) {
    extern __shared__ float dyn[];
    float a[CH], b[CH], acc[CH], acc2[CH];
    if (threadIdx.x < 64) dyn[threadIdx.x] = in[threadIdx.x];
    __syncthreads();
#pragma unroll
    for (int c = 0; c < CH; c++) {
        a[c] = in[threadIdx.x + c * 256];
        b[c] = in[threadIdx.x + (8 + c) * 256];
        acc[c] = 0.f;
        acc2[c] = 0.f;
    }
    const unsigned long long t0 = __builtin_amdgcn_s_memtime(), r0 = __builtin_amdgcn_s_memrealtime();
    for (int it = 0; it < iters; it++) {
#pragma unroll
        for (int u = 0; u < UNROLL; u++) step<MIX, CH, NOPS>(acc, acc2, a, b, sc, dyn);
    }
    const unsigned long long t1 = __builtin_amdgcn_s_memtime(), r1 = __builtin_amdgcn_s_memrealtime();
    float s = 0;
#pragma unroll
    for (int c = 0; c < CH; c++) s += acc[c] + acc2[c];
    out[blockIdx.x * 256 + threadIdx.x] = s;
    if (blockIdx.x == 0 && threadIdx.x == 0) {
        clk[0] = t1 - t0;
        clk[1] = r1 - r0;
    }
}

static float *g_out, *g_in;
static unsigned long long* g_clk;
static int g_cus = 256;

template <int MIX, int CH, int NOPS = 0>
void run_case(int waves) {
    constexpr int NI_RAW = MIX == P8_FWD ? 4 : (MIX == P8_BWD || MIX == P8_BWD_V || MIX == P8_BWD_LDS) ? 7 : MIX == INF ? 3 : MIX == BOUND ? 4 : MIX == GENP ? 5 : MIX == GENP_BWD ? 7 : 1;
    constexpr int UNROLL = (128 / (CH * NI_RAW)) > 0 ? (128 / (CH * NI_RAW)) : 1;
    auto kern = mix_kernel<MIX, CH, UNROLL, NOPS>;
    const int blocks = g_cus * waves;
    // LDS per workgroup: exactly `waves` workgroups fit a compute unit (160 KB)
    // (allocation granularity is coarse: sizes that are multiples of 8 KB, and of which waves + 1 do not fit)
    static const int kLdsKb[9] = {0, 160, 80, 48, 40, 32, 24, 20, 16};
    const int lds = kLdsKb[waves] * 1024;
    CHECK(hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, lds));
    const double per_iter = (double)CH * NI_RAW * UNROLL;  // wave instructions per loop iteration
    const int iters = (int)(3.0e6 / per_iter / waves) + 1; // about 3 M wave instructions per SIMD: ~3 ms
    hipEvent_t e0, e1;
    CHECK(hipEventCreate(&e0));
    CHECK(hipEventCreate(&e1));
    kern<<<blocks, 256, lds>>>(g_out, g_in, iters / 10 + 1, 1.0f, g_clk);
    CHECK(hipEventRecord(e0));
    kern<<<blocks, 256, lds>>>(g_out, g_in, iters, 1.0f, g_clk);
    CHECK(hipEventRecord(e1));
    CHECK(hipEventSynchronize(e1));
    CHECK(hipGetLastError());
    float ms = 0;
    CHECK(hipEventElapsedTime(&ms, e0, e1));
    unsigned long long clk[2];
    CHECK(hipMemcpy(clk, g_clk, sizeof(clk), hipMemcpyDeviceToHost));
    const double instr = (double)blocks * 4 * iters * per_iter;        // wave-level vector instructions
    const double cyc = ms * 1e-3 * 2.4e9 * (g_cus * 4.0);               // SIMD cycles available at 2.4 GHz
    // s_memrealtime ticks at 100 MHz; when s_memtime ticks differently it is the shader clock
    const double mhz = clk[1] > 0 ? (double)clk[0] / (double)clk[1] * 100.0 : 0.0;
    const bool shader_clock = mhz > 150.0;
    const double cpi = cyc / instr;
    printf("%-48s nops=%d chains=%d waves/simd=%d  %6.3f ms  %6.2f cyc/instr", kMix[MIX].name, NOPS, CH, waves, ms, cpi);
    if (shader_clock) printf("  clock %4.0f MHz  %6.2f real cyc/instr", mhz, cpi * mhz / 2400.0);
    if (kMix[MIX].pairs > 0) printf("  %6.2f cyc/pair", cpi * kMix[MIX].instr / kMix[MIX].pairs);
    printf("\n");
    fflush(stdout);
    CHECK(hipEventDestroy(e0));
    CHECK(hipEventDestroy(e1));
}

template <int MIX>
void run_mix() {
    for (int w : {1, 2, 3, 4, 5, 6, 8}) {
        run_case<MIX, 1>(w);
        run_case<MIX, 2>(w);
        run_case<MIX, 4>(w);
        run_case<MIX, 8>(w);
    }
}

// the same with one to four idle cycles (s_nop) after every vector instruction: does a wave that issues less often
// leave the SIMD a better schedule?
template <int MIX>
void run_mix_nops() {
    for (int w : {2, 3, 4, 5, 6, 8}) {
        run_case<MIX, 1, 1>(w); run_case<MIX, 2, 1>(w); run_case<MIX, 4, 1>(w); run_case<MIX, 8, 1>(w);
        run_case<MIX, 1, 2>(w); run_case<MIX, 2, 2>(w); run_case<MIX, 4, 2>(w); run_case<MIX, 8, 2>(w);
        run_case<MIX, 1, 3>(w); run_case<MIX, 2, 3>(w); run_case<MIX, 4, 3>(w); run_case<MIX, 8, 3>(w);
        run_case<MIX, 1, 4>(w); run_case<MIX, 2, 4>(w); run_case<MIX, 4, 4>(w); run_case<MIX, 8, 4>(w);
    }
}

template <int MIX>
void dispatch(int want) {
    if (want < 0 || want == MIX) run_mix<MIX>();
    if constexpr (MIX + 1 < NMIX) dispatch<MIX + 1>(want);
}

int main(int argc, char** argv) {
    hipDeviceProp_t prop;
    CHECK(hipGetDeviceProperties(&prop, 0));
    g_cus = prop.multiProcessorCount;
    int wall_khz = 0;
    (void)hipDeviceGetAttribute(&wall_khz, hipDeviceAttributeWallClockRate, 0);
    printf("device: %s, %d CUs, clockRate %d kHz, wall clock %d kHz\n", prop.name, g_cus, prop.clockRate, wall_khz);
    CHECK(hipMalloc(&g_out, (size_t)g_cus * 8 * 256 * 4));
    CHECK(hipMalloc(&g_in, 256 * 16 * 4));
    {
        // operands in [0.5, 1.5): realistic switching activity (an all-zero data path draws less power)
        float h[256 * 16];
        unsigned r = 12345u;
        for (int i = 0; i < 256 * 16; i++) {
            r = r * 1664525u + 1013904223u;
            h[i] = 0.5f + (float)(r >> 8) / 16777216.0f;
        }
        CHECK(hipMemcpy(g_in, h, sizeof(h), hipMemcpyHostToDevice));
    }
    CHECK(hipMalloc(&g_clk, 16));
    if (argc <= 1) dispatch<0>(-1);
    for (int i = 1; i < argc; i++) {
        if (argv[i][0] == 'n') {  // "n": the idle-cycle sweep of the three mixes that model the p = 8 kernels
            run_mix_nops<MUL>();
            run_mix_nops<P8_FWD>();
            run_mix_nops<P8_BWD>();
        } else {
            dispatch<0>(atoi(argv[i]));
        }
    }
    return 0;
}
