// igs_common.h -- compile-time tunables and small device helpers shared by all kernels.
// Included by igs_gs2d.hip inside its anonymous namespace (one translation unit).
#pragma once


constexpr float kNegHalfLog2e = -0.72134752044448170368f;  // -0.5 * log2(e)
constexpr int kThreads = 256;

// Tunables (compile-time; -D overrides exist so that variants can be timed against each other).
// The defaults are the fastest of the timed settings at B=16, N=8192, 256x256, C=3.
#ifndef IGS_FWD_SEP_P
#define IGS_FWD_SEP_P 16
#endif
#ifndef IGS_BWD_G
#define IGS_BWD_G 2
#endif
#ifndef IGS_FWD_WAVES
#define IGS_FWD_WAVES 8
#endif
#ifndef IGS_FWD_MAX_SPLIT
#define IGS_FWD_MAX_SPLIT 64
#endif
#ifndef IGS_BWD_WAVES
#define IGS_BWD_WAVES 16
#endif
// rows per lane in the separable forward: as many as the accumulator VGPRs (P x (C+1)) allow
__host__ __device__ constexpr int fwd_sep_p(int C) { return C <= 3 ? IGS_FWD_SEP_P : (C <= 8 ? 8 : 4); }
// pixels per lane, general forward
__host__ __device__ constexpr int fwd_gen_p(int C) { return C <= 4 ? 8 : 4; }
// Gaussians per lane, general backward (more independent chains per pixel record)
#ifndef IGS_BWD_GEN_G
#define IGS_BWD_GEN_G 4
#endif
__host__ __device__ constexpr int bwd_gen_g(int C) { return C <= 4 ? IGS_BWD_GEN_G : 2; }
// Gaussians per lane, separable backward: two independent chains per pixel record where the sums of two
// fit in registers (C <= 4); with wide colour vectors one (B=4, N=32768, 384x640, C=16: 3.38 -> 3.08 ms)
__host__ __device__ constexpr int bwd_sep_g(int C) { return C <= 4 ? IGS_BWD_G : 1; }

__host__ __device__ constexpr int rec_stride_of(int C) { return (6 + C + 3) & ~3; }
__host__ __device__ constexpr int pix_stride_sep(int C) { return (C + 1 + 3) & ~3; }
__host__ __device__ constexpr int pix_stride_gen(int C) { return (C + 3 + 3) & ~3; }

__device__ __forceinline__ float hw_exp2(float v) { return __builtin_amdgcn_exp2f(v); }

// Workgroups are dealt round-robin to the 8 XCDs (each with its own L2).  Map the linear
// block id so that every XCD walks one contiguous range of tiles (same image -> the same
// packed Gaussian records stay hot in that XCD's L2).  Launch 8*ceil(total/8) blocks and
// skip results >= total.
__device__ __forceinline__ int xcd_contiguous(int linear, int total) {
    const int per = (total + 7) >> 3;
    return (linear & 7) * per + (linear >> 3);
}
