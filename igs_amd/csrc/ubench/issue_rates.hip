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
    CK(hipFree(out));
    CK(hipFree(in));
    CK(hipFree(clk));
    return 0;
}
