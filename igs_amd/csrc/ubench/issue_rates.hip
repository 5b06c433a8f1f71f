// issue_rates.hip -- instruction issue rates of one gfx950 SIMD, measured.
//
// Stand-alone program (no library code): the figures it prints are the ceilings the splat and
// diversity-loss kernels are priced against beside the published peak.  Every kernel reads the
// shader clock (clock64) and the 100 MHz wall clock (wall_clock64) around its loop, so a rate is
// reported in cycles of the clock the device actually ran at, not of a nominal one.
//
//   section 1  fp32 VALU ops with VGPR-only operands: cycles per wave instruction and SIMD as a
//              function of the distance between dependent instructions in a wave's stream
//              (1 = a back-to-back chain) and of the resident waves per SIMD
//   section 2  v_exp_f32 alone and interleaved with fused multiply-adds
//   section 3  v_mfma_f32_32x32x2_f32: an endless accumulation chain, chains that restart from
//              zero every KH steps (a tile loop), and the same with the 16 results consumed by
//              v_max_f32 (what a nearest-neighbour search does per tile)
//   section 4  matrix-core and vector instructions sharing a SIMD
//   section 5  v_fmac_f32 with its three operands in distinct / shared register banks
//
// Build: hipcc -O3 --offload-arch=gfx950 -Xclang -target-feature -Xclang -packed-fp32-ops issue_rates.hip
#include <hip/hip_runtime.h>

#include <cstdio>
#include <cstdlib>

#define CK(x)                                                                          \
    do {                                                                               \
        hipError_t e_ = (x);                                                           \
        if (e_ != hipSuccess) {                                                        \
            std::printf("HIP error %s at line %d\n", hipGetErrorString(e_), __LINE__); \
            std::exit(1);                                                              \
        }                                                                              \
    } while (0)

namespace {

typedef float v16f __attribute__((ext_vector_type(16)));
constexpr int kIters = 2048;
constexpr int kCus = 256;

struct Timing {
    float ms;
    double mhz;  // shader clock during the launch
};

// Launches `kernel` twice (the first run warms clocks and caches) on wgs workgroups of 256 lanes.
template <class K, class... A>
Timing timed(K kernel, int wgs, size_t lds, long long* clk, A... args) {
    hipEvent_t e0, e1;
    CK(hipEventCreate(&e0));
    CK(hipEventCreate(&e1));
    hipLaunchKernelGGL(kernel, dim3(wgs), dim3(256), lds, 0, args..., clk);
    CK(hipDeviceSynchronize());
    CK(hipEventRecord(e0));
    hipLaunchKernelGGL(kernel, dim3(wgs), dim3(256), lds, 0, args..., clk);
    CK(hipEventRecord(e1));
    CK(hipDeviceSynchronize());
    Timing t;
    CK(hipEventElapsedTime(&t.ms, e0, e1));
    long long c[2];
    CK(hipMemcpy(c, clk, sizeof(c), hipMemcpyDeviceToHost));
    t.mhz = c[1] ? c[0] / (c[1] * 0.01) : 0.0;
    CK(hipEventDestroy(e0));
    CK(hipEventDestroy(e1));
    return t;
}

__device__ inline void stamp(long long* clk, long long t0, long long w0) {
    const long long t1 = clock64(), w1 = wall_clock64();
    if (blockIdx.x == 0 && threadIdx.x == 0) {
        clk[0] = t1 - t0;
        clk[1] = w1 - w0;
    }
}

// ----------------------------------------------------------------------------- section 1
// DIST independent accumulators updated round robin: a wave's next instruction on the same
// register is DIST instructions away.  OP: 0 v_fmac, 1 v_mul, 2 v_add, 3 v_fma (3 sources).
template <int DIST, int OP>
__global__ __launch_bounds__(256) void k_valu(float* out, long long* clk) {
    extern __shared__ float lds[];
    float a[16];
#pragma unroll
    for (int j = 0; j < 16; ++j) a[j] = threadIdx.x * 0.001f + j;
    float x = threadIdx.x * 1e-3f + 0.5f, y = 0.999f;
    asm volatile("" : "+v"(x), "+v"(y));
    const long long t0 = clock64(), w0 = wall_clock64();
    for (int i = 0; i < kIters; ++i) {
#pragma unroll
        for (int r = 0; r < 64 / DIST; ++r) {
#pragma unroll
            for (int j = 0; j < DIST; ++j) {
                if (OP == 0) asm volatile("v_fmac_f32 %0, %1, %2" : "+v"(a[j]) : "v"(x), "v"(y));
                if (OP == 1) asm volatile("v_mul_f32 %0, %0, %1" : "+v"(a[j]) : "v"(y));
                if (OP == 2) asm volatile("v_add_f32 %0, %0, %1" : "+v"(a[j]) : "v"(y));
                if (OP == 3) asm volatile("v_fma_f32 %0, %0, %1, %2" : "+v"(a[j]) : "v"(y), "v"(x));
            }
        }
    }
    stamp(clk, t0, w0);
    float r = 0;
#pragma unroll
    for (int j = 0; j < 16; ++j) r += a[j];
    out[blockIdx.x * 256 + threadIdx.x] = r + lds[0] * 0.0f;
}

// LDS per workgroup sized so that `waves` workgroups (one wave per SIMD each) fit a CU's 160 KB
// and one more does not (1 KB of slack for the allocation granularity).
size_t lds_for(int waves) {
    size_t lds = (size_t)(160 * 1024 / waves - 1024) & ~(size_t)255;
    return lds > 65536 ? 65536 : lds;
}

template <int DIST, int OP>
void run_valu(int waves, float* out, long long* clk) {
    static const char* names[] = {"v_fmac_f32", "v_mul_f32", "v_add_f32", "v_fma_f32"};
    CK(hipFuncSetAttribute((const void*)k_valu<DIST, OP>, hipFuncAttributeMaxDynamicSharedMemorySize, 65536));
    const Timing t = timed(k_valu<DIST, OP>, kCus * waves, lds_for(waves), clk, out);
    const double n = (double)kIters * 64 * waves;  // wave instructions per SIMD
    std::printf("%-11s distance %2d  waves/SIMD %d  %7.3f ms  clock %4.0f MHz  %5.2f cycles per wave instruction and SIMD\n",
                names[OP], DIST, waves, t.ms, t.mhz, t.ms * 1e-3 * t.mhz * 1e6 / n);
}

// ----------------------------------------------------------------------------- section 2
// Per step: one v_exp_f32 and NF v_fmac_f32, eight independent chains (distance 8).
template <int NF>
__global__ __launch_bounds__(256) void k_exp(float* out, long long* clk) {
    float t[8], a[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) {
        t[j] = -(threadIdx.x * 0.001f + j);
        a[j] = threadIdx.x * 0.002f + j;
    }
    float x = 0.5f, y = 0.999f;
    asm volatile("" : "+v"(x), "+v"(y));
    const long long t0 = clock64(), w0 = wall_clock64();
    for (int i = 0; i < kIters; ++i) {
#pragma unroll
        for (int r = 0; r < 4; ++r) {
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                asm volatile("v_exp_f32 %0, %0" : "+v"(t[j]));
#pragma unroll
                for (int f = 0; f < NF; ++f) asm volatile("v_fmac_f32 %0, %1, %2" : "+v"(a[j]) : "v"(x), "v"(y));
            }
        }
    }
    stamp(clk, t0, w0);
    float r = 0;
#pragma unroll
    for (int j = 0; j < 8; ++j) r += t[j] + a[j];
    out[blockIdx.x * 256 + threadIdx.x] = r;
}

template <int NF>
void run_exp(int waves, float* out, long long* clk) {
    const Timing t = timed(k_exp<NF>, kCus * waves, 0, clk, out);
    const double n = (double)kIters * 32 * waves;  // exps per SIMD
    const double cyc = t.ms * 1e-3 * t.mhz * 1e6 / n;
    std::printf("v_exp_f32 + %d v_fmac_f32  waves/SIMD %d  %7.3f ms  clock %4.0f MHz  %5.2f cycles per group, %5.2f per instruction\n",
                NF, waves, t.ms, t.mhz, cyc, cyc / (1 + NF));
}

// ----------------------------------------------------------------------------- section 3
// MODE 0: one endless chain; 1: restart from zero every KH steps, results unused;
// 2: restart and fold the 16 results of a tile into a running maximum (16 v_max_f32).
template <int KH, int MODE>
__global__ __launch_bounds__(256) void k_mfma(float* out, const float* in, long long* clk) {
    float a[KH], b[KH];
    for (int t = 0; t < KH; ++t) {
        a[t] = in[threadIdx.x + 64 * t];
        b[t] = in[threadIdx.x + 64 * t + 1];
    }
    float r = 0;
    v16f keep = {0};
    const long long t0 = clock64(), w0 = wall_clock64();
    for (int i = 0; i < kIters; ++i) {
        v16f acc = {0};
        for (int t = 0; t < KH; ++t) asm volatile("" : "+v"(a[t]));  // nothing is hoisted out of the loop
        if (MODE == 0) acc = keep;
#pragma unroll
        for (int t = 0; t < KH; ++t) acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a[t], b[t], acc, 0, 0, 0);
        if (MODE == 0) keep = acc;
        if (MODE == 1) asm volatile("" ::"v"(acc));
        if (MODE == 2)
            for (int q = 0; q < 16; ++q) r = fmaxf(r, acc[q]);
    }
    stamp(clk, t0, w0);
    for (int q = 0; q < 16; ++q) r += keep[q];
    out[blockIdx.x * 256 + threadIdx.x] = r;
}

template <int KH, int MODE>
void run_mfma(int waves, float* out, const float* in, long long* clk) {
    static const char* names[] = {"endless chain", "restart every KH", "restart + 16 v_max"};
    const Timing t = timed(k_mfma<KH, MODE>, kCus * waves, 0, clk, out, in);
    const double n = (double)kIters * KH * waves;  // matrix instructions per SIMD
    const double flop = n * 1024 * 4096.0;
    std::printf("mfma_f32_32x32x2  KH %2d  %-18s waves/SIMD %d  %7.3f ms  clock %4.0f MHz  %6.2f cycles per mfma  %6.1f TFLOP/s\n",
                KH, names[MODE], waves, t.ms, t.mhz, t.ms * 1e-3 * t.mhz * 1e6 / n, flop / t.ms / 1e9);
}

// ----------------------------------------------------------------------------- section 4
// Per step and wave: one mfma_f32_32x32x2 (chains of 8 that restart) and NV independent
// v_fmac_f32.  If vector instructions issued in the shadow of the 16-pass matrix instruction the
// time per step would stay at the matrix instruction's until NV is large.
template <int NV>
__global__ __launch_bounds__(256) void k_mix(float* out, const float* in, long long* clk) {
    float a[8], b[8], v[8];
    for (int t = 0; t < 8; ++t) {
        a[t] = in[threadIdx.x + 64 * t];
        b[t] = in[threadIdx.x + 64 * t + 1];
        v[t] = threadIdx.x * 0.001f + t;
    }
    float x = 0.5f, y = 0.999f, r = 0;
    asm volatile("" : "+v"(x), "+v"(y));
    const long long t0 = clock64(), w0 = wall_clock64();
    for (int i = 0; i < kIters; ++i) {
        v16f acc = {0};
        for (int t = 0; t < 8; ++t) asm volatile("" : "+v"(a[t]));
#pragma unroll
        for (int t = 0; t < 8; ++t) {
            acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a[t], b[t], acc, 0, 0, 0);
#pragma unroll
            for (int f = 0; f < NV; ++f) asm volatile("v_fmac_f32 %0, %1, %2" : "+v"(v[(t + f) & 7]) : "v"(x), "v"(y));
        }
        asm volatile("" ::"v"(acc));
    }
    stamp(clk, t0, w0);
    for (int t = 0; t < 8; ++t) r += v[t];
    out[blockIdx.x * 256 + threadIdx.x] = r;
}

template <int NV>
void run_mix(int waves, float* out, const float* in, long long* clk) {
    const Timing t = timed(k_mix<NV>, kCus * waves, 0, clk, out, in);
    const double n = (double)kIters * 8 * waves;  // steps per SIMD
    std::printf("1 mfma_f32_32x32x2 + %d v_fmac_f32  waves/SIMD %d  %7.3f ms  clock %4.0f MHz  %6.2f cycles per step\n", NV,
                waves, t.ms, t.mhz, t.ms * 1e-3 * t.mhz * 1e6 / n);
}


// ----------------------------------------------------------------------------- section 5
// Register banks.  The accumulation phase of the separable forward is 64 x `v_fmac_f32 acc, e, coef`
// per record: 16 weights e (each used four times in a row), 4 coefficients, 64 accumulators.  A VGPR's
// bank is its index mod 4.  The same 64 instructions with three register assignments (all below v120,
// so four waves fit a SIMD): no two operands of an instruction in one bank; the two sources (e, coef) of
// every instruction in one bank; and the assignment the compiler chose for k_fwd_sep<3,16> (its
// registers renumbered, banks kept: 16 instructions with both sources in one bank, 26 more with the
// accumulator in the bank of a source).
#define FM(acc, e, c) "v_fmac_f32 v" #acc ", v" #e ", v" #c "\n"
#define BANKS_FREE \
    FM(5, 3, 0) FM(6, 3, 1) FM(8, 3, 2) FM(9, 3, 4) \
    FM(10, 7, 0) FM(12, 7, 1) FM(13, 7, 2) FM(14, 7, 4) \
    FM(17, 11, 0) FM(16, 11, 1) FM(20, 11, 2) FM(18, 11, 4) \
    FM(21, 15, 0) FM(22, 15, 1) FM(24, 15, 2) FM(25, 15, 4) \
    FM(26, 19, 0) FM(28, 19, 1) FM(29, 19, 2) FM(30, 19, 4) \
    FM(33, 23, 0) FM(32, 23, 1) FM(36, 23, 2) FM(34, 23, 4) \
    FM(37, 27, 0) FM(38, 27, 1) FM(40, 27, 2) FM(41, 27, 4) \
    FM(42, 31, 0) FM(44, 31, 1) FM(45, 31, 2) FM(46, 31, 4) \
    FM(49, 35, 0) FM(48, 35, 1) FM(52, 35, 2) FM(50, 35, 4) \
    FM(53, 39, 0) FM(54, 39, 1) FM(56, 39, 2) FM(57, 39, 4) \
    FM(58, 43, 0) FM(60, 43, 1) FM(61, 43, 2) FM(62, 43, 4) \
    FM(65, 47, 0) FM(64, 47, 1) FM(68, 47, 2) FM(66, 47, 4) \
    FM(69, 51, 0) FM(70, 51, 1) FM(72, 51, 2) FM(73, 51, 4) \
    FM(74, 55, 0) FM(76, 55, 1) FM(77, 55, 2) FM(78, 55, 4) \
    FM(81, 59, 0) FM(80, 59, 1) FM(84, 59, 2) FM(82, 59, 4) \
    FM(85, 63, 0) FM(86, 63, 1) FM(88, 63, 2) FM(89, 63, 4)
#define BANKS_SOURCES_COLLIDE \
    FM(0, 3, 67) FM(1, 3, 71) FM(2, 3, 75) FM(4, 3, 79) \
    FM(5, 7, 67) FM(6, 7, 71) FM(8, 7, 75) FM(9, 7, 79) \
    FM(10, 11, 67) FM(12, 11, 71) FM(13, 11, 75) FM(14, 11, 79) \
    FM(16, 15, 67) FM(17, 15, 71) FM(18, 15, 75) FM(20, 15, 79) \
    FM(21, 19, 67) FM(22, 19, 71) FM(24, 19, 75) FM(25, 19, 79) \
    FM(26, 23, 67) FM(28, 23, 71) FM(29, 23, 75) FM(30, 23, 79) \
    FM(32, 27, 67) FM(33, 27, 71) FM(34, 27, 75) FM(36, 27, 79) \
    FM(37, 31, 67) FM(38, 31, 71) FM(40, 31, 75) FM(41, 31, 79) \
    FM(42, 35, 67) FM(44, 35, 71) FM(45, 35, 75) FM(46, 35, 79) \
    FM(48, 39, 67) FM(49, 39, 71) FM(50, 39, 75) FM(52, 39, 79) \
    FM(53, 43, 67) FM(54, 43, 71) FM(56, 43, 75) FM(57, 43, 79) \
    FM(58, 47, 67) FM(60, 47, 71) FM(61, 47, 75) FM(62, 47, 79) \
    FM(64, 51, 67) FM(65, 51, 71) FM(66, 51, 75) FM(68, 51, 79) \
    FM(69, 55, 67) FM(70, 55, 71) FM(72, 55, 75) FM(73, 55, 79) \
    FM(74, 59, 67) FM(76, 59, 71) FM(77, 59, 75) FM(78, 59, 79) \
    FM(80, 63, 67) FM(81, 63, 71) FM(82, 63, 75) FM(84, 63, 79)
#define BANKS_COMPILER \
    FM(2, 0, 1) FM(5, 0, 6) FM(4, 0, 3) FM(7, 0, 8) \
    FM(10, 9, 1) FM(13, 9, 6) FM(11, 9, 3) FM(14, 9, 8) \
    FM(12, 15, 1) FM(16, 15, 6) FM(19, 15, 3) FM(17, 15, 8) \
    FM(23, 20, 1) FM(27, 20, 6) FM(18, 20, 3) FM(21, 20, 8) \
    FM(22, 25, 1) FM(26, 25, 6) FM(29, 25, 3) FM(31, 25, 8) \
    FM(33, 30, 1) FM(24, 30, 6) FM(35, 30, 3) FM(34, 30, 8) \
    FM(37, 28, 1) FM(32, 28, 6) FM(39, 28, 3) FM(38, 28, 8) \
    FM(41, 45, 1) FM(36, 45, 6) FM(43, 45, 3) FM(42, 45, 8) \
    FM(49, 46, 1) FM(40, 46, 6) FM(47, 46, 3) FM(50, 46, 8) \
    FM(53, 51, 1) FM(44, 51, 6) FM(55, 51, 3) FM(54, 51, 8) \
    FM(57, 48, 1) FM(52, 48, 6) FM(59, 48, 3) FM(58, 48, 8) \
    FM(61, 56, 1) FM(63, 56, 6) FM(62, 56, 3) FM(65, 56, 8) \
    FM(67, 69, 1) FM(66, 69, 6) FM(73, 69, 3) FM(60, 69, 8) \
    FM(70, 74, 1) FM(77, 74, 6) FM(64, 74, 3) FM(71, 74, 8) \
    FM(81, 75, 1) FM(68, 75, 6) FM(79, 75, 3) FM(85, 75, 8) \
    FM(72, 78, 1) FM(82, 78, 6) FM(89, 78, 3) FM(76, 78, 8)
#define CLOBBER_V0_V119                                                                                        \
    "v0", "v1", "v2", "v3", "v4", "v5", "v6", "v7", "v8", "v9", "v10", "v11", "v12", "v13", "v14", "v15", "v16", \
        "v17", "v18", "v19", "v20", "v21", "v22", "v23", "v24", "v25", "v26", "v27", "v28", "v29", "v30", "v31", \
        "v32", "v33", "v34", "v35", "v36", "v37", "v38", "v39", "v40", "v41", "v42", "v43", "v44", "v45", "v46", \
        "v47", "v48", "v49", "v50", "v51", "v52", "v53", "v54", "v55", "v56", "v57", "v58", "v59", "v60", "v61", \
        "v62", "v63", "v64", "v65", "v66", "v67", "v68", "v69", "v70", "v71", "v72", "v73", "v74", "v75", "v76", \
        "v77", "v78", "v79", "v80", "v81", "v82", "v83", "v84", "v85", "v86", "v87", "v88", "v89", "v90", "v91", \
        "v92", "v93", "v94", "v95", "v96", "v97", "v98", "v99", "v100", "v101", "v102", "v103", "v104", "v105",  \
        "v106", "v107", "v108", "v109", "v110", "v111", "v112", "v113", "v114", "v115", "v116", "v117", "v118",  \
        "v119"

// The loop runs kIters times inside one asm statement (registers hold whatever they held: the
// timing of v_fmac_f32 does not depend on the values).
#define BANK_KERNEL(NAME, BODY)                                                                            \
    __global__ __launch_bounds__(256) void NAME(float* out, long long* clk) {                              \
        extern __shared__ float lds[];                                                                     \
        const long long t0 = clock64(), w0 = wall_clock64();                                               \
        asm volatile("s_mov_b32 s20, 2048\n"                                                               \
                     "1:\n" BODY "s_sub_u32 s20, s20, 1\n"                                                 \
                     "s_cmp_lg_u32 s20, 0\n"                                                               \
                     "s_cbranch_scc1 1b\n" ::                                                              \
                         : CLOBBER_V0_V119, "s20", "scc");                                                 \
        stamp(clk, t0, w0);                                                                                \
        out[blockIdx.x * 256 + threadIdx.x] = lds[0];                                                      \
    }
BANK_KERNEL(k_banks_free, BANKS_FREE)
BANK_KERNEL(k_banks_sources, BANKS_SOURCES_COLLIDE)
BANK_KERNEL(k_banks_compiler, BANKS_COMPILER)

template <class K>
void run_banks(K kernel, const char* name, int waves, float* out, long long* clk) {
    const Timing t = timed(kernel, kCus * waves, lds_for(waves), clk, out);
    const double n = (double)kIters * 64 * waves;
    std::printf("%-44s waves/SIMD %d  %7.3f ms  clock %4.0f MHz  %5.2f cycles per v_fmac_f32 and SIMD\n", name, waves, t.ms,
                t.mhz, t.ms * 1e-3 * t.mhz * 1e6 / n);
}

}  // namespace

int main() {
    hipDeviceProp_t prop;
    CK(hipGetDeviceProperties(&prop, 0));
    std::printf("device %s (%s), %d CUs, clockRate attribute %d kHz\n", prop.name, prop.gcnArchName,
                prop.multiProcessorCount, prop.clockRate);
    if (prop.multiProcessorCount != kCus) std::printf("note: the grids assume %d CUs\n", kCus);
    float *out, *in;
    long long* clk;
    CK(hipMalloc(&out, sizeof(float) * 256 * kCus * 8));
    CK(hipMalloc(&in, 4 * 65536));
    CK(hipMemset(in, 0, 4 * 65536));
    CK(hipMalloc(&clk, 16));

    std::printf("\n== 1. fp32 VALU, VGPR operands\n");
    for (int w : {1, 2, 3, 4, 8}) {
        run_valu<1, 0>(w, out, clk);
        run_valu<2, 0>(w, out, clk);
        run_valu<4, 0>(w, out, clk);
        run_valu<8, 0>(w, out, clk);
        run_valu<16, 0>(w, out, clk);
    }
    for (int w : {3, 8}) {
        run_valu<1, 1>(w, out, clk);
        run_valu<4, 1>(w, out, clk);
        run_valu<1, 2>(w, out, clk);
        run_valu<4, 2>(w, out, clk);
        run_valu<1, 3>(w, out, clk);
        run_valu<4, 3>(w, out, clk);
    }
    std::printf("\n== 2. v_exp_f32\n");
    for (int w : {3, 8}) {
        run_exp<0>(w, out, clk);
        run_exp<3>(w, out, clk);
        run_exp<7>(w, out, clk);
        run_exp<14>(w, out, clk);
    }
    std::printf("\n== 3. fp32 matrix cores\n");
    for (int w : {1, 2, 4}) {
        run_mfma<6, 0>(w, out, in, clk);
        run_mfma<6, 1>(w, out, in, clk);
        run_mfma<6, 2>(w, out, in, clk);
        run_mfma<16, 1>(w, out, in, clk);
        run_mfma<16, 2>(w, out, in, clk);
    }
    std::printf("\n== 4. matrix and vector instructions on one SIMD\n");
    for (int w : {1, 4}) {
        run_mix<0>(w, out, in, clk);
        run_mix<2>(w, out, in, clk);
        run_mix<4>(w, out, in, clk);
        run_mix<8>(w, out, in, clk);
        run_mix<16>(w, out, in, clk);
    }
    std::printf("\n== 5. register banks: 64 x v_fmac_f32 acc, e, coef per step\n");
    for (int w : {2, 3, 4}) {
        run_banks(k_banks_free, "no two operands in one bank", w, out, clk);
        run_banks(k_banks_compiler, "the compiler's assignment in k_fwd_sep<3,16>", w, out, clk);
        run_banks(k_banks_sources, "both sources in one bank", w, out, clk);
    }
    CK(hipFree(out));
    CK(hipFree(in));
    CK(hipFree(clk));
    return 0;
}
