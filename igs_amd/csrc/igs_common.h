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
#ifndef IGS_FWD_WAVES
#define IGS_FWD_WAVES 8
#endif
#ifndef IGS_FWD_MAX_SPLIT
#define IGS_FWD_MAX_SPLIT 64
#endif
// (backward: four waves per SIMD wanted; only small problems are split further than the 32-row tiles that
// keep the lists short: B=1 N=2048 256x256 fit step 159 / 145 / 141 / 145 us with 16 / 8 / 4 / 2)
#ifndef IGS_BWD_WAVES
#define IGS_BWD_WAVES 4
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
// Gaussians per lane, separable backward: one (a tile's last group of list positions is half empty on
// average, and its idle lanes cost more with two per lane than sharing the pixel records' reads saves)
__host__ __device__ constexpr int bwd_sep_g(int) { return 1; }

__host__ __device__ constexpr int rec_stride_of(int C) { return (6 + C + 3) & ~3; }
// Records of the separable kernels (see sep_terms): the forward's px, py, sD, skD, A'', alpha,
// alpha*c_0.., tag, A', B2', D' (none for C > 8: with four rows per lane the hoisted part of the completed square
// costs what it saves, and that forward reads the plain records); the backward's sA, skA, D'', tag.
#ifndef IGS_FWD_SQUARE
#define IGS_FWD_SQUARE 1
#endif
__host__ __device__ constexpr bool fwd_square(int C) { return IGS_FWD_SQUARE && fwd_sep_p(C) >= 8; }
__host__ __device__ constexpr int frec_stride_of(int C) { return fwd_square(C) ? (10 + C + 3) & ~3 : 0; }
constexpr int kBrecStride = 4;
// The completed square is evaluated in coordinates relative to the middle of a lane's rows (forward) or
// of a tile's columns (backward); its rounding grows with s times the largest such coordinate (s = sD, sA:
// the square's scale; an error of about 1e-7 s |y'| |u| in the exponent), so where that product exceeds a
// limit (Gaussians sharper than the pixel spacing, grids whose coordinates jump within a tile) the pair is
// evaluated term by term instead.  The forward, whose result is held to 1e-6, chooses per wave and record
// (wave-uniform, so the other evaluation costs one instruction per pair more and nothing else) with a
// tight limit; the backward chooses per lane, where a wave with lanes of both kinds runs both loops, and
// its sums are held to 1e-4 of the largest: its limit only catches what would be inaccurate beyond that.
#ifndef IGS_SEP_LIMIT_FWD
#define IGS_SEP_LIMIT_FWD 8.0f
#endif
#ifndef IGS_SEP_LIMIT_BWD
#define IGS_SEP_LIMIT_BWD 64.0f
#endif
constexpr float kSepSpanLimitFwd = IGS_SEP_LIMIT_FWD;
constexpr float kSepSpanLimitBwd = IGS_SEP_LIMIT_BWD;
// floats of the packed buffer per (padded) Gaussian: record, bin record, forward and backward records
// of the separable kernels
__host__ __device__ constexpr int packed_floats_per_gaussian(int C) {
    return rec_stride_of(C) + 8 + frec_stride_of(C) + kBrecStride;
}
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
// The same with the XCD's range walked from another starting tile (`rot` tiles further on, cyclically).
__device__ __forceinline__ int xcd_contiguous_from(int linear, int total, int rot) {
    const int per = (total + 7) >> 3;
    return (linear & 7) * per + ((linear >> 3) + rot) % per;
}
