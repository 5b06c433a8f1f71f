// igs_gs2d.hip -- hand-written gfx950 (CDNA4) kernels and the C ABI for the 2-D Gaussian
// splatting forward/backward.
//
// Math (reference src/igs/gs2d.py:24-44): q = A dx^2 + 2 B dx dy + D dy^2,
// e = exp(-q/2), w = alpha e, out_c = sum_n w c_nc / (sum_n w + eps).
//
// Design in one paragraph.  The path is bound by fp32 VALU + transcendental issue, not by
// HBM (a few tens of MB per call) and not by MFMA (colour contraction has C = 3), so the
// kernels are organised to need no cross-lane reduction at all and the fewest, cheapest
// VALU instructions per (Gaussian, pixel) pair:
//   * forward  : a lane owns pixels, the Gaussian record is wave-uniform; den and the C
//                numerators stay in VGPRs for the whole Gaussian loop.
//   * backward : a lane owns Gaussians, the pixel record (g^ = g/(den+eps), -s = -<g^,out>)
//                is wave-uniform; the lane accumulates the six moments of G e and the C
//                colour sums over its pixel tile in VGPRs.  Per-tile partials go to a
//                [B,T,6+C,N] buffer which a finalize kernel sums in a fixed order (no
//                float atomics anywhere, bit-reproducible).
//   * the wave-uniform record stream goes global -> LDS (cooperative, double-buffered) ->
//     VGPRs (broadcast ds_read_b128), because on gfx950 a VALU op with VGPR-only operands
//     issues almost twice as fast as one with an SGPR operand.
//   * separable grids (x independent of the row, y independent of the column: every
//     linspace grid) let both kernels hoist the row/column part of the quadratic form and
//     of the moment sums: 3 VALU ops per pair for q instead of 7, 5 instead of 9 for the
//     moments.
// exp() is one v_exp_f32: A, 2B, D are pre-multiplied by -0.5 log2(e) when packed.
// Record arrays are zero-padded (alpha = 0 / g^ = 0 records contribute exactly 0) so the hot
// loops have no tails.
//
// Build flags disable packed-fp32 instruction selection (-packed-fp32-ops), so every VALU
// op below is a scalar-per-lane fp32 op.

#include <hip/hip_runtime.h>

#include <stdint.h>
#include <stdlib.h>

#include "igs_hip.h"

namespace {

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
#ifndef IGS_BWD_WAVES
#define IGS_BWD_WAVES 16
#endif
// rows per lane in the separable forward: as many as the accumulator VGPRs (P x (C+1)) allow
__host__ __device__ constexpr int fwd_sep_p(int C) { return C <= 3 ? IGS_FWD_SEP_P : (C <= 8 ? 8 : 4); }
// pixels per lane, general forward
__host__ __device__ constexpr int fwd_gen_p(int C) { return C <= 4 ? 8 : 4; }
// Gaussians per lane, general backward (more independent chains per pixel record)
__host__ __device__ constexpr int bwd_gen_g(int C) { return C <= 4 ? 4 : 2; }
constexpr int kBwdG = IGS_BWD_G;  // Gaussians per lane, backward

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

// ----------------------------------------------------------------------------- pack
// Reach box of a Gaussian: the axis-aligned bounding box of the ellipse q <= kReachQ, outside
// of which its weight is exactly zero in these kernels: there the exponent
// q' = -0.5 log2(e) q is below -160, ten binades under the -149/-150 at which exp2 returns 0
// in fp32 whatever the denormal mode (the margin covers the rounding of q' itself, which is
// a few ulp of its largest term).  Pixels outside the box therefore receive exactly +0 from
// this Gaussian and give exactly 0 to its gradient sums, so skipping them changes no bit.
// Half extents: sqrt(kReachQ Sigma_xx), sqrt(kReachQ Sigma_yy) with Sigma the covariance that
// (A, B, D) invert.  A record with a non-finite field or a non-positive-definite (A, B, D)
// gets an unbounded box (its NaN/inf must propagate as without culling); padding records get
// an empty one.  Stored as (xlo, xhi, ylo, yhi).
constexpr double kReachQ = 160.0 / 0.72134752044448170368;

__device__ __forceinline__ float4 reach_box(float px, float py, double sxx, double syy, bool bounded) {
    const float inf = __builtin_inff();
    if (!bounded || !(sxx >= 0.0) || !(syy >= 0.0) || !isfinite(px) || !isfinite(py))
        return make_float4(-inf, inf, -inf, inf);
    // rounded outwards: one part in 1e5 is far more than the fp32 rounding of the bounds
    const double hx = sqrt(kReachQ * sxx) * 1.00001, hy = sqrt(kReachQ * syy) * 1.00001;
    const double ax = fabs((double)px) * 1e-6 + 1e-30, ay = fabs((double)py) * 1e-6 + 1e-30;
    return make_float4((float)((double)px - hx - ax), (float)((double)px + hx + ax),
                       (float)((double)py - hy - ay), (float)((double)py + hy + ay));
}

__device__ __forceinline__ float4 empty_box() {
    const float inf = __builtin_inff();
    return make_float4(inf, -inf, inf, -inf);
}

// One thread per record.  Record: px, py, A', B2', D', alpha, alpha*c_0.. (padded to x4)
// with A' = k A, B2' = 2 k B, D' = k D, k = -0.5 log2 e.  Records N..Np-1 are zero.
// The reach boxes [B][Np] follow the records in the packed buffer.
template <bool kScaleRot>
__global__ __launch_bounds__(kThreads) void k_pack(const float* __restrict__ position,
                                                   const float* __restrict__ p0,  // cov00 | scales
                                                   const float* __restrict__ p1,  // cov01 | rotations
                                                   const float* __restrict__ p2,  // cov11 | unused
                                                   const float* __restrict__ alphas,
                                                   const float* __restrict__ colors, int N,
                                                   int Np, int C, int RS, float eps,
                                                   float* __restrict__ packed,
                                                   float4* __restrict__ boxes, int cull) {
    const int n = blockIdx.x * kThreads + threadIdx.x;
    const int b = blockIdx.y;
    if (n >= Np) return;
    float* r = packed + ((size_t)b * Np + n) * RS;
    if (n >= N) {  // padding: alpha = 0 and e = exp2(0) = 1, so it contributes exactly 0
        for (int c = 0; c < RS; ++c) r[c] = 0.0f;
        boxes[(size_t)b * Np + n] = empty_box();
        return;
    }
    const size_t i = (size_t)b * N + n;
    // The closed form runs in fp64 and is rounded once: an error of a few fp32 ulp in A', B2', D'
    // would be multiplied by |q| (tens, for sharp Gaussians) in the exponent.  O(BN) work.
    double A, Bc, D, sxx, syy;
    bool bounded;
    if (kScaleRot) {
        const double s0 = p0[2 * i], s1 = p0[2 * i + 1];
        double sn, cs;
        sincos((double)p1[i], &sn, &cs);
        const double v0 = s0 * s0 + (double)eps, v1 = s1 * s1 + (double)eps;
        const double i0 = 1.0 / v0, i1 = 1.0 / v1;
        A = cs * cs * i0 + sn * sn * i1;
        Bc = cs * sn * (i0 - i1);
        D = sn * sn * i0 + cs * cs * i1;
        sxx = cs * cs * v0 + sn * sn * v1;
        syy = sn * sn * v0 + cs * cs * v1;
        bounded = v0 > 0.0 && v1 > 0.0;
    } else {
        A = p0[i];
        Bc = p1[i];
        D = p2[i];
        const double det = A * D - Bc * Bc;
        bounded = A > 0.0 && det > 0.0;
        sxx = D / det;
        syy = A / det;
    }
    constexpr double k = -0.72134752044448170368;  // -0.5 * log2(e)
    const float al = alphas[i];
    const float px = position[2 * i], py = position[2 * i + 1];
    r[0] = px;
    r[1] = py;
    r[2] = (float)(k * A);
    r[3] = (float)(2.0 * k * Bc);
    r[4] = (float)(k * D);
    r[5] = al;
    bool fin = isfinite(al) && isfinite(r[2]) && isfinite(r[3]) && isfinite(r[4]);
    for (int c = 0; c < C; ++c) {
        const float v = al * colors[i * C + c];
        r[6 + c] = v;
        fin = fin && isfinite(v) && isfinite(colors[i * C + c]);
    }
    for (int c = 6 + C; c < RS; ++c) r[c] = 0.0f;
    boxes[(size_t)b * Np + n] = reach_box(px, py, sxx, syy, cull && bounded && fin);
}

// Module head fused into the pack: reads gs_feature rows [px, py, log_s0, log_s1, theta,
// opacity logit (unused), c_0..c_{C-1}] (reference src/igs/gs2d.py:635-644) and applies the
// module's activations scales = exp(log_s) + eps, alpha = 1 (src/igs/gs2d.py:673-675), plus
// an optional position offset (pos_map_offset, src/igs/gs2d.py:654-667).  Also writes the raw
// colours [B][N][Cp] (zero-padded to the kernels' channel count) that the backward reads.
__global__ __launch_bounds__(kThreads) void k_pack_feature(const float* __restrict__ feat,
                                                           const float* __restrict__ pos_off, int N,
                                                           int Np, int C, int Cp, int RS, float eps,
                                                           float* __restrict__ packed,
                                                           float4* __restrict__ boxes,
                                                           float* __restrict__ colors_out, int cull) {
    const int n = blockIdx.x * kThreads + threadIdx.x;
    const int b = blockIdx.y;
    if (n >= Np) return;
    float* r = packed + ((size_t)b * Np + n) * RS;
    if (n >= N) {
        for (int c = 0; c < RS; ++c) r[c] = 0.0f;
        boxes[(size_t)b * Np + n] = empty_box();
        return;
    }
    const size_t i = (size_t)b * N + n;
    const float* f = feat + i * (6 + C);
    const double s0 = (double)expf(f[2]) + (double)eps, s1 = (double)expf(f[3]) + (double)eps;
    double sn, cs;
    sincos((double)f[4], &sn, &cs);
    const double v0 = s0 * s0 + (double)eps, v1 = s1 * s1 + (double)eps;
    const double i0 = 1.0 / v0, i1 = 1.0 / v1;
    const double A = cs * cs * i0 + sn * sn * i1;
    const double Bc = cs * sn * (i0 - i1);
    const double D = sn * sn * i0 + cs * cs * i1;
    constexpr double k = -0.72134752044448170368;
    float px = f[0], py = f[1];
    if (pos_off) {
        px += pos_off[2 * i];
        py += pos_off[2 * i + 1];
    }
    r[0] = px;
    r[1] = py;
    r[2] = (float)(k * A);
    r[3] = (float)(2.0 * k * Bc);
    r[4] = (float)(k * D);
    r[5] = 1.0f;
    bool fin = isfinite(r[2]) && isfinite(r[3]) && isfinite(r[4]);
    for (int c = 0; c < Cp; ++c) {
        const float col = c < C ? f[6 + c] : 0.0f;
        r[6 + c] = col;
        colors_out[i * Cp + c] = col;
        fin = fin && isfinite(col);
    }
    for (int c = 6 + Cp; c < RS; ++c) r[c] = 0.0f;
    boxes[(size_t)b * Np + n] = reach_box(px, py, cs * cs * v0 + sn * sn * v1, sn * sn * v0 + cs * cs * v1,
                                          cull && fin && v0 > 0.0 && v1 > 0.0);
}

// ----------------------------------------------------------------------------- binning
// Per pixel tile, the Gaussians whose reach box meets the tile's coordinate range, as a list
// of indices in increasing order (so that sums over a list keep the order of the unculled
// sum), and the count.  One workgroup per (tile, image) scans all N boxes; positions come
// from ballots and a fixed-order prefix over the four waves, so the lists are reproducible.
// With `slots` set, the inverse map is written as well: slots[b][tile][n] = position of
// Gaussian n in the tile's list, or -1 when it is not listed (every n < N is written).
// Separable grids only: a tile is tile_w columns x tile_h rows and its coordinate range is
// [min, max] of x over its columns and of y over its rows (no monotonicity assumed).
struct BinArgs {
    const float4* boxes;  // [B][Np]
    const float* x;
    const float* y;
    long sxb, sxw, syb, syh;
    int N, Np, H, W;
    int tile_w, tile_h, tiles_x, tiles_y;
    int* counts;  // [B][tiles]
    int* lists;   // [B][tiles][Np]
    int* slots;   // [B][tiles][Np] or nullptr
    const int* flag;
    int want;
};

constexpr int kBinThreads = 1024, kBinWaves = kBinThreads / 64;  // many loads in flight per tile

__global__ __launch_bounds__(kBinThreads) void k_bin(const BinArgs a) {
    if (a.flag != nullptr && *a.flag != a.want) return;
    __shared__ float red[4][kBinThreads];
    __shared__ int wsum[kBinWaves];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int tiles = a.tiles_x * a.tiles_y;
    const int t = blockIdx.x, b = blockIdx.y;
    const int ty = t / a.tiles_x, tx = t - ty * a.tiles_x;
    const int c0 = tx * a.tile_w, c1 = min(a.W, c0 + a.tile_w);
    const int r0 = ty * a.tile_h, r1 = min(a.H, r0 + a.tile_h);
    const float inf = __builtin_inff();
    float xlo = inf, xhi = -inf, ylo = inf, yhi = -inf;
    bool bad = false;
    for (int c = c0 + tid; c < c1; c += kBinThreads) {
        const float v = a.x[b * a.sxb + (long)c * a.sxw];
        bad = bad || !(v == v);
        xlo = fminf(xlo, v);
        xhi = fmaxf(xhi, v);
    }
    for (int r = r0 + tid; r < r1; r += kBinThreads) {
        const float v = a.y[b * a.syb + (long)r * a.syh];
        bad = bad || !(v == v);
        ylo = fminf(ylo, v);
        yhi = fmaxf(yhi, v);
    }
    if (bad) {  // a NaN coordinate: nothing may be culled for this tile
        xlo = ylo = -inf;
        xhi = yhi = inf;
    }
    red[0][tid] = xlo;
    red[1][tid] = -xhi;
    red[2][tid] = ylo;
    red[3][tid] = -yhi;
    __syncthreads();
    for (int k = kBinThreads / 2; k > 0; k >>= 1) {
        if (tid < k) {
#pragma unroll
            for (int f = 0; f < 4; ++f) red[f][tid] = fminf(red[f][tid], red[f][tid + k]);
        }
        __syncthreads();
    }
    const float txlo = red[0][0], txhi = -red[1][0], tylo = red[2][0], tyhi = -red[3][0];
    int* list = a.lists + ((size_t)b * tiles + t) * a.Np;
    int* slot = a.slots ? a.slots + ((size_t)b * tiles + t) * a.Np : nullptr;
    const float4* boxes = a.boxes + (size_t)b * a.Np;
    // Each wave scans one contiguous share of the Gaussians twice, without barriers: first to
    // count, then (with the shares' counts prefixed in wave order) to write.
    const int per_wave = ((a.N + kBinWaves - 1) / kBinWaves + 63) & ~63;
    const int nb = wave * per_wave, ne = min(a.N, nb + per_wave);
    const unsigned long long below = (1ull << lane) - 1ull;
    // kU boxes per lane are loaded together, so that kU loads are in flight instead of one
    constexpr int kU = 8;
    auto classify = [&](int n0, bool (&listed)[kU], bool (&in)[kU]) {
        float4 bb[kU];
#pragma unroll
        for (int u = 0; u < kU; ++u) {
            const int n = n0 + u * 64 + lane;
            bb[u] = boxes[min(n, a.N - 1)];
        }
#pragma unroll
        for (int u = 0; u < kU; ++u) {
            in[u] = n0 + u * 64 + lane < ne;
            // "definitely outside" negated, so that NaN bounds count as inside
            listed[u] = in[u] && !(bb[u].y < txlo || bb[u].x > txhi || bb[u].w < tylo || bb[u].z > tyhi);
        }
    };
    int cnt = 0;
    for (int n0 = nb; n0 < ne; n0 += 64 * kU) {
        bool listed[kU], in[kU];
        classify(n0, listed, in);
#pragma unroll
        for (int u = 0; u < kU; ++u) cnt += __popcll(__ballot(listed[u]));
    }
    if (lane == 0) wsum[wave] = cnt;
    __syncthreads();
    int base = 0, total = 0;
#pragma unroll
    for (int w = 0; w < kBinWaves; ++w) {
        if (w < wave) base += wsum[w];
        total += wsum[w];
    }
    for (int n0 = nb; n0 < ne; n0 += 64 * kU) {
        bool listed[kU], in[kU];
        classify(n0, listed, in);
#pragma unroll
        for (int u = 0; u < kU; ++u) {
            const int n = n0 + u * 64 + lane;
            const unsigned long long m = __ballot(listed[u]);
            const int pos = base + __popcll(m & below);
            if (listed[u]) list[pos] = n;
            if (slot != nullptr && in[u]) slot[n] = listed[u] ? pos : -1;
            base += __popcll(m);
        }
    }
    if (tid == 0) a.counts[(size_t)b * tiles + t] = total;
}

// ----------------------------------------------------------------------------- forward
struct FwdArgs {
    const float* packed;  // [B][Np][RS]
    const float* x;
    const float* y;
    long sxb, sxh, sxw, syb, syh, syw;
    int B, Np, H, W;
    int n_per_split, S;  // n_per_split % 4 == 0
    int tiles_x, tiles_y, total_tiles, wx;
    float eps;
    float* out;
    float* den;
    float* part;  // [S][B][C+1][HW] when S > 1
    const int* counts;  // separable: Gaussians listed per tile [B][tiles]
    const int* lists;   // separable: their indices [B][tiles][Np]
    const int* flag;  // AUTO grid mode: run only if *flag == want (nullptr: always run)
    int want;
};

// AUTO grid mode launches both the separable and the general variant of a kernel; the
// device-side classification flag (1 = separable) decides which one does the work.
#define IGS_GATE(a) \
    if ((a).flag != nullptr && *(a).flag != (a).want) return

// On gfx950 a fp32 VALU op whose operands are all VGPRs (or literals) issues about every
// 2.2-2.7 cycles per wave64, while any SGPR operand makes it a 4-cycle op (measured; the
// constant bus broadcast is the slow part).  So wave-uniform operands are NOT fed from SGPRs:
// the uniform record stream (Gaussians in the forward, pixels in the backward) goes
// global -> LDS (cooperatively, double-buffered) -> VGPRs through broadcast ds_read_b128
// (every lane reads the same address: conflict-free), and the hot loops contain VGPR-only
// VALU instructions plus LDS reads that issue on their own port.
template <int C>
struct GRec {
    float px, py, A, B2, D, al;
    float ac[C];
};

// Unpacks one record held in R4 float4 registers (read from a wave-uniform LDS address).
template <int C>
__device__ __forceinline__ GRec<C> lds_grec(const float4* r) {
    constexpr int R4 = rec_stride_of(C) / 4;
    float v[4 * R4];
#pragma unroll
    for (int i = 0; i < R4; ++i) {
        const float4 t = r[i];
        v[4 * i] = t.x;
        v[4 * i + 1] = t.y;
        v[4 * i + 2] = t.z;
        v[4 * i + 3] = t.w;
    }
    GRec<C> g;
    g.px = v[0];
    g.py = v[1];
    g.A = v[2];
    g.B2 = v[3];
    g.D = v[4];
    g.al = v[5];
#pragma unroll
    for (int c = 0; c < C; ++c) g.ac[c] = v[6 + c];
    return g;
}

// Keeps a wave-uniform value in a VGPR (an empty asm the compiler cannot see through), so that
// instructions using it stay VGPR-only.
__device__ __forceinline__ float in_vgpr(float v) {
    asm volatile("" : "+v"(v));
    return v;
}

#ifndef IGS_GCHUNK
#define IGS_GCHUNK 64
#endif
#ifndef IGS_PCHUNK
#define IGS_PCHUNK 256
#endif
#ifndef IGS_STREAM_UNROLL
#define IGS_STREAM_UNROLL 2
#endif
constexpr int kStreamUnroll = IGS_STREAM_UNROLL;  // records whose LDS reads are in flight together
constexpr int kGaussChunk = IGS_GCHUNK;  // Gaussian records per LDS buffer

// Streams `count` records of R4 float4 each from global memory to every wave of the
// workgroup through the double-buffered LDS window sh[2][CH*R4]; body(const float4* rec) runs
// once per record with a wave-uniform LDS pointer.  Records past `count` in the last chunk
// read as all-zero (for a Gaussian record: alpha = 0, adds exactly 0).  Must be called by all
// kThreads threads of the workgroup (it contains barriers).
// With kGather, record i of the stream is src record index[i] (a tile's Gaussian list).
template <int R4, int CH, bool kGather = false, class Body>
__device__ __forceinline__ void stream_records_lds(const float4* __restrict__ src, int count,
                                                   float4* sh, Body&& body,
                                                   const int* __restrict__ index = nullptr) {
    constexpr int E = CH * R4;                          // float4 per chunk
    constexpr int PRE = (E + kThreads - 1) / kThreads;  // float4 per thread per chunk
    const int total = count * R4;
    const int chunks = (count + CH - 1) / CH;
    const int tid = threadIdx.x;
    const float4 zero = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
    // Gather: the record indices of a chunk are loaded one chunk before its records, so that
    // no load in the loop waits for another load.
    int idx[PRE];
    auto load_idx = [&](int chunk) {
#pragma unroll
        for (int i = 0; i < PRE; ++i) {
            const int e = i * kThreads + tid, ge = chunk * E + e;
            idx[i] = (kGather && e < E && ge < total) ? index[ge / R4] : 0;
        }
    };
    float4 pre[PRE];
    auto load_records = [&](int chunk) {
#pragma unroll
        for (int i = 0; i < PRE; ++i) {
            const int e = i * kThreads + tid, ge = chunk * E + e;
            const bool valid = e < E && ge < total;
            if (kGather)
                pre[i] = valid ? src[(size_t)idx[i] * R4 + (ge % R4)] : zero;
            else
                pre[i] = valid ? src[ge] : zero;
        }
    };
    load_idx(0);
    load_records(0);
    load_idx(1);
#pragma unroll
    for (int i = 0; i < PRE; ++i) {
        const int e = i * kThreads + tid;
        if (e < E) sh[e] = pre[i];
    }
    __syncthreads();
    for (int k = 0; k < chunks; ++k) {
        if (k + 1 < chunks) {
            load_records(k + 1);
            load_idx(k + 2);
        }
        const float4* cur = sh + (k & 1) * E;
        // The LDS reads of kStreamUnroll records are issued together and pinned above the work
        // (the compiler would otherwise sink each read next to its first use and wait for it
        // there); each record's body then only waits for its own reads, so one LDS latency is
        // exposed per group instead of per record.
#pragma unroll 1
        for (int n = 0; n < CH; n += kStreamUnroll) {
            float4 rr[kStreamUnroll][R4];
#pragma unroll
            for (int u = 0; u < kStreamUnroll; ++u)
#pragma unroll
                for (int i = 0; i < R4; ++i) rr[u][i] = cur[(n + u) * R4 + i];
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int u = 0; u < kStreamUnroll; ++u) {
                body(rr[u]);
                __builtin_amdgcn_sched_barrier(0);
            }
        }
        if (k + 1 < chunks) {
            float4* nxt = sh + ((k + 1) & 1) * E;
#pragma unroll
            for (int i = 0; i < PRE; ++i) {
                const int e = i * kThreads + tid;
                if (e < E) nxt[e] = pre[i];
            }
        }
        __syncthreads();
    }
}

template <int C>
__device__ __forceinline__ void fwd_store(const FwdArgs& a, int b, int s, int p, float dsum,
                                          const float (&num)[C]) {
    const size_t HW = (size_t)a.H * a.W;
    if (a.S == 1) {
        const float inv = 1.0f / (dsum + a.eps);
        a.den[(size_t)b * HW + p] = dsum;
#pragma unroll
        for (int c = 0; c < C; ++c) a.out[((size_t)b * C + c) * HW + p] = num[c] * inv;
    } else {
        float* dst = a.part + ((size_t)s * a.B + b) * (C + 1) * HW + p;
#pragma unroll
        for (int c = 0; c < C; ++c) dst[(size_t)c * HW] = num[c];
        dst[(size_t)C * HW] = dsum;
    }
}

// Separable grid: lane = one column, P consecutive rows; wave = 64 columns x P rows;
// workgroup = wx x (4/wx) waves, all four streaming the same Gaussians.  Per Gaussian and
// lane: dx, A'dx^2, B2'dx once, then per pixel dy, 2 fma, exp2, 1 + C fma.
template <int C, int P>
__global__ __launch_bounds__(kThreads) void k_fwd_sep(const FwdArgs a) {
    constexpr int RS = rec_stride_of(C), R4 = RS / 4;
    __shared__ float4 sh[2 * kGaussChunk * R4];
    IGS_GATE(a);
    const int tile = xcd_contiguous(blockIdx.x, a.total_tiles);
    if (tile >= a.total_tiles) return;  // workgroup-uniform
    const int per_img = a.tiles_x * a.tiles_y;
    const int b = tile / per_img;
    const int tl = tile - b * per_img;
    const int ty = tl / a.tiles_x, tx = tl - ty * a.tiles_x;
    const int wave = threadIdx.x >> 6;
    const int lane = threadIdx.x & 63;
    const int wxi = wave % a.wx, wyi = wave / a.wx;
    const int col = (tx * a.wx + wxi) * 64 + lane;
    const int row0 = (ty * (4 / a.wx) + wyi) * P;
    const float xv = a.x[b * a.sxb + (long)min(col, a.W - 1) * a.sxw];
    float yv[P];
#pragma unroll
    for (int p = 0; p < P; ++p) yv[p] = in_vgpr(a.y[b * a.syb + (long)min(row0 + p, a.H - 1) * a.syh]);

    float dsum[P], num[P][C];
#pragma unroll
    for (int p = 0; p < P; ++p) {
        dsum[p] = 0.0f;
#pragma unroll
        for (int c = 0; c < C; ++c) num[p][c] = 0.0f;
    }
    // this tile's Gaussians (those whose reach box meets it), split S ways by list position
    const int s = blockIdx.y;
    const int count = a.counts[(size_t)b * per_img + tl];
    const int per = ((count + a.S - 1) / a.S + 3) & ~3;
    const int n0 = min(count, s * per);
    const int n1 = min(count, n0 + per);
    const int* list = a.lists + ((size_t)b * per_img + tl) * a.Np + n0;
    const float4* src = reinterpret_cast<const float4*>(a.packed + (size_t)b * a.Np * RS);
    stream_records_lds<R4, kGaussChunk, true>(src, n1 - n0, sh, [&](const float4* r) {
        const GRec<C> g = lds_grec<C>(r);
        const float dx = xv - g.px;
        const float adx = g.A * dx;
        const float c0 = adx * dx;
        const float c1 = g.B2 * dx;
        // three phases, so that the P independent chains overlap their latencies and the
        // transcendental ops issue back to back
        float e[P];
#pragma unroll
        for (int p = 0; p < P; ++p) {
            const float dy = yv[p] - g.py;
            const float t = fmaf(g.D, dy, c1);
            e[p] = fmaf(t, dy, c0);
        }
#pragma unroll
        for (int p = 0; p < P; ++p) e[p] = hw_exp2(e[p]);
#pragma unroll
        for (int p = 0; p < P; ++p) {
            dsum[p] = fmaf(e[p], g.al, dsum[p]);
#pragma unroll
            for (int c = 0; c < C; ++c) num[p][c] = fmaf(e[p], g.ac[c], num[p][c]);
        }
    }, list);
    if (col < a.W) {
#pragma unroll
        for (int p = 0; p < P; ++p)
            if (row0 + p < a.H) fwd_store<C>(a, b, s, (row0 + p) * a.W + col, dsum[p], num[p]);
    }
}

// General grid: lane = P pixels of a flat 256*P pixel tile.
template <int C, int P>
__global__ __launch_bounds__(kThreads) void k_fwd_gen(const FwdArgs a) {
    constexpr int RS = rec_stride_of(C), R4 = RS / 4;
    __shared__ float4 sh[2 * kGaussChunk * R4];
    IGS_GATE(a);
    const int tile = xcd_contiguous(blockIdx.x, a.total_tiles);
    if (tile >= a.total_tiles) return;  // workgroup-uniform
    const int per_img = a.tiles_x;
    const int b = tile / per_img;
    const int tl = tile - b * per_img;
    const int HW = a.H * a.W;
    float xv[P], yv[P];
    int pix[P];
#pragma unroll
    for (int j = 0; j < P; ++j) {
        pix[j] = tl * (kThreads * P) + j * kThreads + (int)threadIdx.x;
        const int pc = min(pix[j], HW - 1);
        const int h = pc / a.W, w = pc - h * a.W;
        xv[j] = a.x[b * a.sxb + h * a.sxh + w * a.sxw];
        yv[j] = a.y[b * a.syb + h * a.syh + w * a.syw];
    }
    float dsum[P], num[P][C];
#pragma unroll
    for (int j = 0; j < P; ++j) {
        dsum[j] = 0.0f;
#pragma unroll
        for (int c = 0; c < C; ++c) num[j][c] = 0.0f;
    }
    const int s = blockIdx.y;
    const int n0 = s * a.n_per_split;
    const int n1 = min(a.Np, n0 + a.n_per_split);
    const float4* src = reinterpret_cast<const float4*>(a.packed + ((size_t)b * a.Np + n0) * RS);
    stream_records_lds<R4, kGaussChunk>(src, n1 - n0, sh, [&](const float4* r) {
        const GRec<C> g = lds_grec<C>(r);
        float e[P];
#pragma unroll
        for (int j = 0; j < P; ++j) {
            const float dx = xv[j] - g.px;
            const float dy = yv[j] - g.py;
            float t = g.A * dx;
            t = fmaf(g.B2, dy, t);
            const float v = g.D * dy;
            float q = t * dx;
            e[j] = fmaf(v, dy, q);
        }
#pragma unroll
        for (int j = 0; j < P; ++j) e[j] = hw_exp2(e[j]);
#pragma unroll
        for (int j = 0; j < P; ++j) {
            dsum[j] = fmaf(e[j], g.al, dsum[j]);
#pragma unroll
            for (int c = 0; c < C; ++c) num[j][c] = fmaf(e[j], g.ac[c], num[j][c]);
        }
    });
#pragma unroll
    for (int j = 0; j < P; ++j)
        if (pix[j] < HW) fwd_store<C>(a, b, s, pix[j], dsum[j], num[j]);
}

// Split-N combine: fixed-order sum over the S partial images, then normalise.
__global__ __launch_bounds__(kThreads) void k_fwd_combine(const float* __restrict__ part, int S,
                                                          int B, int C, int HW, float eps,
                                                          float* __restrict__ out,
                                                          float* __restrict__ den,
                                                          const int* __restrict__ flag, int want) {
    if (flag != nullptr && *flag != want) return;
    const int p = blockIdx.x * kThreads + threadIdx.x;
    const int b = blockIdx.y;
    if (p >= HW) return;
    float d = 0.0f;
    for (int s = 0; s < S; ++s) d += part[(((size_t)s * B + b) * (C + 1) + C) * HW + p];
    den[(size_t)b * HW + p] = d;
    const float inv = 1.0f / (d + eps);
    for (int c = 0; c < C; ++c) {
        float v = 0.0f;
        for (int s = 0; s < S; ++s) v += part[(((size_t)s * B + b) * (C + 1) + c) * HW + p];
        out[((size_t)b * C + c) * HW + p] = v * inv;
    }
}

// ----------------------------------------------------------------------------- backward
// Prologue, one thread per (padded) pixel: g^_c = g_c / (den + eps), s = <g^, out>.
//   separable: records [B][H][Wp][CP] = g^_0..g^_{C-1}, -s, 0..; columns W..Wp-1 are zero
//              records; followed by the compact column coordinates xs [B][Wp]
//              (padding columns repeat x of column W-1).
//   general  : records [B][HWp][CP] = x, y, g^.., -s, 0..; padding pixels are zero records
//              carrying the coordinates of the last pixel.
// With `target` set (fit step), the upstream gradient is that of a mean-squared-error loss,
// g_c = gscale (out_c - target_c), formed here instead of being read from `gout`, and each
// workgroup writes its sum of (out - target)^2 (fixed-order LDS sum) to
// loss_part[b * gridDim.x + blockIdx.x].
template <int C, bool kSep>
__global__ __launch_bounds__(kThreads) void k_bwd_pix(const float* __restrict__ out,
                                                      const float* __restrict__ den,
                                                      const float* __restrict__ gout,
                                                      const float* __restrict__ target,
                                                      float gscale,
                                                      float* __restrict__ loss_part,
                                                      const float* __restrict__ x,
                                                      const float* __restrict__ y, long sxb,
                                                      long sxh, long sxw, long syb, long syh,
                                                      long syw, int B, int H, int W, int Wp,
                                                      int HWp, float eps,
                                                      float* __restrict__ pixrec,
                                                      const int* __restrict__ flag, int want) {
    constexpr int CP = kSep ? pix_stride_sep(C) : pix_stride_gen(C);
    constexpr int OFF = kSep ? 0 : 2;
    if (flag != nullptr && *flag != want) return;
    const int HW = H * W;
    const int i = blockIdx.x * kThreads + threadIdx.x;  // padded pixel index
    const int b = blockIdx.y;
    int h = 0, w = 0;
    bool valid, inside;  // inside: this thread owns a (padded) record; valid: a real pixel
    if (kSep) {
        inside = i < H * Wp;
        h = inside ? i / Wp : 0;
        w = inside ? i - h * Wp : 0;
        valid = inside && w < W;
        if (inside && h == 0) {
            float* xs = pixrec + (size_t)B * H * Wp * CP;
            xs[(size_t)b * Wp + w] = x[b * sxb + (long)min(w, W - 1) * sxw];
        }
    } else {
        inside = i < HWp;
        valid = i < HW;
        const int pc = min(i, HW - 1);
        h = pc / W;
        w = pc - h * W;
    }
    float r[CP];
#pragma unroll
    for (int k = 0; k < CP; ++k) r[k] = 0.0f;
    float sq = 0.0f;
    if (valid) {
        const int p = h * W + w;
        const float inv = 1.0f / (den[(size_t)b * HW + p] + eps);
        float s = 0.0f;
#pragma unroll
        for (int c = 0; c < C; ++c) {
            const size_t idx = ((size_t)b * C + c) * HW + p;
            const float o = out[idx];
            float g;
            if (target != nullptr) {
                const float d = o - target[idx];
                sq = fmaf(d, d, sq);
                g = gscale * d;
            } else {
                g = gout[idx];
            }
            const float gh = g * inv;
            s = fmaf(gh, o, s);
            r[OFF + c] = gh;
        }
        r[OFF + C] = -s;
    }
    if (inside) {
        if (!kSep) {
            r[0] = x[b * sxb + h * sxh + w * sxw];
            r[1] = y[b * syb + h * syh + w * syw];
        }
        const size_t rec = kSep ? ((size_t)b * H * Wp + i) : ((size_t)b * HWp + i);
        float4* dst = reinterpret_cast<float4*>(pixrec + rec * CP);
#pragma unroll
        for (int k = 0; k < CP / 4; ++k)
            dst[k] = make_float4(r[4 * k], r[4 * k + 1], r[4 * k + 2], r[4 * k + 3]);
    }
    if (loss_part != nullptr) {  // kernel-argument uniform: every thread reaches the barriers
        __shared__ float red[kThreads];
        red[threadIdx.x] = sq;
        __syncthreads();
        for (int k = kThreads / 2; k > 0; k >>= 1) {
            if ((int)threadIdx.x < k) red[threadIdx.x] += red[threadIdx.x + k];
            __syncthreads();
        }
        if (threadIdx.x == 0) loss_part[(size_t)b * gridDim.x + blockIdx.x] = red[0];
    }
}

// loss = scale * sum(loss_part[0..count)), one workgroup, fixed order.
__global__ __launch_bounds__(kThreads) void k_loss_sum(const float* __restrict__ loss_part, int count,
                                                       float scale, float* __restrict__ loss,
                                                       const int* __restrict__ flag, int want) {
    if (flag != nullptr && *flag != want) return;
    __shared__ float red[kThreads];
    float s = 0.0f;
    for (int i = threadIdx.x; i < count; i += kThreads) s += loss_part[i];
    red[threadIdx.x] = s;
    __syncthreads();
    for (int k = kThreads / 2; k > 0; k >>= 1) {
        if ((int)threadIdx.x < k) red[threadIdx.x] += red[threadIdx.x + k];
        __syncthreads();
    }
    if (threadIdx.x == 0) *loss = red[0] * scale;
}

// ----------------------------------------------------------------------------- AdamW
// Decoupled-weight-decay Adam over one flat parameter block, the update of torch.optim.AdamW
// (amsgrad off) as the fit script configures it (scripts/2dgs_img_comp.py:186-193).  The
// step counter and learning rate live in device memory so that a captured graph advances:
//   state = {lr, t, 1 - beta1^t, sqrt(1 - beta2^t)}; lr is written by the host, the rest by
// k_adamw_tick (one thread, powers in double).
__global__ void k_adamw_tick(float* __restrict__ state, float beta1, float beta2) {
    if (threadIdx.x != 0 || blockIdx.x != 0) return;
    const float t = state[1] + 1.0f;
    state[1] = t;
    state[2] = (float)(1.0 - pow((double)beta1, (double)t));
    state[3] = (float)sqrt(1.0 - pow((double)beta2, (double)t));
}

__global__ __launch_bounds__(kThreads) void k_adamw(float* __restrict__ param,
                                                    const float* __restrict__ grad,
                                                    float* __restrict__ exp_avg,
                                                    float* __restrict__ exp_avg_sq, long n,
                                                    const float* __restrict__ state, float beta1,
                                                    float beta2, float eps, float weight_decay) {
    const long i = (long)blockIdx.x * kThreads + threadIdx.x;
    if (i >= n) return;
    const float lr = state[0], bc1 = state[2], bc2_sqrt = state[3];
    const float g = grad[i];
    float p = param[i] * (1.0f - lr * weight_decay);
    float m = exp_avg[i];
    m = fmaf(g - m, 1.0f - beta1, m);
    const float v = fmaf(g * g, 1.0f - beta2, exp_avg_sq[i] * beta2);
    const float denom = sqrtf(v) / bc2_sqrt + eps;
    p -= (lr / bc1) * (m / denom);
    param[i] = p;
    exp_avg[i] = m;
    exp_avg_sq[i] = v;
}

struct BwdArgs {
    const float* packed;  // [B][Np][RS]
    const float* colors;  // [B][N][C]
    const float* pixrec;
    const float* xs;      // separable: [B][Wp]
    const float* y;
    long syb, syh;
    int N, Np, H, W, Wp, HWp;
    int per_tile;  // rows (separable) or pixels (general, multiple of 256) per tile
    int T;         // tiles per image (separable: tiles_x * row bands)
    int tiles_x;   // separable: column bands of kBwdTileW columns
    const int* counts;  // separable: Gaussians listed per tile [B][T]
    const int* lists;   // separable: list + complement [B][T][Np]
    float* partial;  // [B][T][6+C][N]
    const int* flag;
    int want;
};

// Partial field order: 0 M0 = sum G e, 1 Mx = sum G e dx, 2 My, 3 Mxx, 4 Mxy, 5 Myy,
// 6+c = sum e g^_c.
// n[g] is the column of the partial array the lane's sums go to (>= N: nothing is stored): the
// Gaussian index on general grids, the position in the tile's list on separable ones.
template <int C, int G>
__device__ __forceinline__ void bwd_store(const BwdArgs& a, int b, int t, const int (&n)[G],
                                          const float (&M)[G][6], const float (&CG)[G][C]) {
    constexpr int NF = 6 + C;
    float* base = a.partial + ((size_t)b * a.T + t) * NF * a.N;
#pragma unroll
    for (int g = 0; g < G; ++g) {
        if (n[g] < a.N) {
#pragma unroll
            for (int f = 0; f < 6; ++f) base[(size_t)f * a.N + n[g]] = M[g][f];
#pragma unroll
            for (int c = 0; c < C; ++c) base[(size_t)(6 + c) * a.N + n[g]] = CG[g][c];
        }
    }
}

// Loads the G Gaussians of this lane; n[g] >= N marks an unused slot (nothing is stored for it).
template <int C, int G>
__device__ __forceinline__ void bwd_load_gaussians(const BwdArgs& a, int b, const int (&n)[G],
                                                   float (&px)[G], float (&py)[G], float (&A)[G],
                                                   float (&B2)[G], float (&D)[G],
                                                   float (&col)[G][C]) {
    constexpr int RS = rec_stride_of(C);
#pragma unroll
    for (int g = 0; g < G; ++g) {
        const int nc = min(n[g], a.N - 1);
        const float* r = a.packed + ((size_t)b * a.Np + nc) * RS;
        px[g] = r[0];
        py[g] = r[1];
        A[g] = r[2];
        B2[g] = r[3];
        D[g] = r[4];
#pragma unroll
        for (int c = 0; c < C; ++c) col[g][c] = a.colors[((size_t)b * a.N + nc) * C + c];
    }
}

// pixel records per LDS buffer; wide records get a shorter chunk so the two buffers stay small
__host__ __device__ constexpr int pix_chunk(int C) { return C <= 4 ? IGS_PCHUNK : 128; }

// columns of a backward pixel tile on separable grids
#ifndef IGS_BWD_MAX_ROWS
#define IGS_BWD_MAX_ROWS 32
#endif
constexpr int kBwdMaxRows = IGS_BWD_MAX_ROWS;
constexpr int kBwdMinRows = 4;
#ifndef IGS_BWD_TILE_W
#define IGS_BWD_TILE_W 64
#endif
constexpr int kBwdTileW = IGS_BWD_TILE_W;

// Separable grid: lane = G Gaussians taken from the tile's list (those whose reach box meets
// the tile; the others are known to get exactly zero from it); the tile is kBwdTileW columns x
// per_tile rows.  Its pixel records stream through LDS in chunks of whole tile rows
// (double-buffered) and are read with broadcast ds_read_b128; the tile's column coordinates sit
// in LDS for the whole kernel.  Per row the dy part of q is hoisted, and row sums
// R0 = sum G e, R1 = sum G e dx, R2 = sum G e dx^2 (and the colour sums) are folded into the
// totals once per row.  A lane's sums are stored at its list position (coalesced); the finalize
// kernel finds them through the tile's slot table and takes 0 for unlisted Gaussians, so tiles
// that a Gaussian does not reach cost neither compute nor memory traffic.
template <int C, int G>
__global__ __launch_bounds__(kThreads) void k_bwd_sep(const BwdArgs a) {
    constexpr int CP = pix_stride_sep(C), CP4 = CP / 4;
    constexpr int PX = pix_chunk(C) > kBwdTileW ? pix_chunk(C) : kBwdTileW;
    constexpr int RPC = PX / kBwdTileW;          // tile rows per chunk
    constexpr int ROW4 = kBwdTileW * CP4;        // float4 per tile row
    constexpr int E = RPC * ROW4;                // float4 per chunk
    constexpr int PRE = (E + kThreads - 1) / kThreads;
    static_assert(PX % kBwdTileW == 0 && RPC >= 1, "chunk must hold whole tile rows");
    __shared__ float4 sh[2 * E];
    __shared__ float4 xsh[kBwdTileW / 4];
    __shared__ float ysh[2][RPC + 1];  // row coordinates of the chunk (+1: read-ahead slot)
    IGS_GATE(a);
    // tiles are the fastest grid dimension: consecutive workgroups (dealt round-robin to the
    // XCDs) then belong to different tiles, and the list-position groups that have work (the
    // low ones) are spread over all XCDs
    const int b = blockIdx.z, t = blockIdx.x, grp = blockIdx.y;
    const int tid = threadIdx.x;
    const int ty = t / a.tiles_x, tx = t - ty * a.tiles_x;
    const int count = a.counts[(size_t)b * a.T + t];
    if (grp * G * kThreads >= count) return;  // workgroup-uniform: no listed Gaussian left
    const int* list = a.lists + ((size_t)b * a.T + t) * a.Np;
    int n[G], slot[G];
#pragma unroll
    for (int g = 0; g < G; ++g) {
        const int pos = (grp * G + g) * kThreads + tid;
        n[g] = pos < count ? list[pos] : a.N;
        slot[g] = pos < count ? pos : a.N;
    }
    float M[G][6], CG[G][C];
#pragma unroll
    for (int g = 0; g < G; ++g) {
#pragma unroll
        for (int f = 0; f < 6; ++f) M[g][f] = 0.0f;
#pragma unroll
        for (int c = 0; c < C; ++c) CG[g][c] = 0.0f;
    }
    float px[G], py[G], A[G], B2[G], D[G], col[G][C];
    bwd_load_gaussians<C, G>(a, b, n, px, py, A, B2, D, col);

    const int c0 = tx * kBwdTileW;
    const int cw = min(a.Wp, c0 + kBwdTileW) - c0;  // columns of this tile, a multiple of 8
    const int r0 = ty * a.per_tile, r1 = min(a.H, r0 + a.per_tile);
    const int chunks = (r1 - r0 + RPC - 1) / RPC;
    const float4 zero = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
    if (tid < kBwdTileW / 4)
        xsh[tid] = 4 * tid < cw ? reinterpret_cast<const float4*>(a.xs + (size_t)b * a.Wp + c0)[tid] : zero;

    // element e of chunk k: float4 (e % ROW4) of tile row (e / ROW4)
    auto fetch = [&](int k, int e) -> float4 {
        const int rr = e / ROW4, rem = e - rr * ROW4;
        const int r = r0 + k * RPC + rr;
        if (r >= r1 || rem >= cw * CP4) return zero;
        const float4* row = reinterpret_cast<const float4*>(a.pixrec + (((size_t)b * a.H + r) * a.Wp + c0) * CP);
        return row[rem];
    };
    // y of tile row (k * RPC + rr), clamped to the tile (the clamped ones are never used)
    auto fetch_y = [&](int k, int rr) -> float {
        return a.y[b * a.syb + (long)min(r0 + k * RPC + rr, r1 - 1) * a.syh];
    };
    float4 pre[PRE];
    float ypre = 0.0f;
#pragma unroll
    for (int i = 0; i < PRE; ++i) {
        const int e = i * kThreads + tid;
        if (e < E) sh[e] = fetch(0, e);
    }
    if (tid <= RPC) ysh[0][tid] = fetch_y(0, min(tid, RPC - 1));
    __syncthreads();

    for (int k = 0; k < chunks; ++k) {
        if (k + 1 < chunks) {
#pragma unroll
            for (int i = 0; i < PRE; ++i) {
                const int e = i * kThreads + tid;
                pre[i] = (e < E) ? fetch(k + 1, e) : zero;
            }
            if (tid <= RPC) ypre = fetch_y(k + 1, min(tid, RPC - 1));
        }
        const float4* cur = sh + (k & 1) * E;
        const float* ycur = ysh[k & 1];
        const int rows = min(RPC, r1 - r0 - k * RPC);
        float ynext = ycur[0];
#pragma unroll 1
        for (int rr = 0; rr < rows; ++rr) {
            // the row coordinate comes from LDS, read one row ahead: a scalar load here would
            // drain the LDS/scalar counter once per tile row
            const float yv = ynext;
            ynext = ycur[rr + 1];
            float dy[G], cyy[G], bdy[G], R0[G], R1[G], R2[G], RC[G][C];
#pragma unroll
            for (int g = 0; g < G; ++g) {
                dy[g] = yv - py[g];
                const float ddy = D[g] * dy[g];
                cyy[g] = ddy * dy[g];
                bdy[g] = B2[g] * dy[g];
                R0[g] = R1[g] = R2[g] = 0.0f;
#pragma unroll
                for (int c = 0; c < C; ++c) RC[g][c] = 0.0f;
            }
            const float4* rowrec = cur + rr * ROW4;
#pragma unroll 1
            for (int i = 0; i < cw; i += 4) {
                const float4 xq = xsh[i >> 2];
                const float xs4[4] = {xq.x, xq.y, xq.z, xq.w};
                // phase 1: exponents of the 4 x G pairs (independent chains)
                float dxs[4][G], ee[4][G];
#pragma unroll
                for (int j = 0; j < 4; ++j)
#pragma unroll
                    for (int g = 0; g < G; ++g) {
                        const float dx = xs4[j] - px[g];
                        const float tt = fmaf(A[g], dx, bdy[g]);
                        ee[j][g] = fmaf(tt, dx, cyy[g]);
                        dxs[j][g] = dx;
                    }
                // phase 2: transcendentals back to back
#pragma unroll
                for (int j = 0; j < 4; ++j)
#pragma unroll
                    for (int g = 0; g < G; ++g) ee[j][g] = hw_exp2(ee[j][g]);
                // phase 3: G = <g^, c> - s and the row sums
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    float pv[CP];
#pragma unroll
                    for (int q4 = 0; q4 < CP4; ++q4) {
                        const float4 tq = rowrec[(i + j) * CP4 + q4];
                        pv[4 * q4] = tq.x;
                        pv[4 * q4 + 1] = tq.y;
                        pv[4 * q4 + 2] = tq.z;
                        pv[4 * q4 + 3] = tq.w;
                    }
#pragma unroll
                    for (int g = 0; g < G; ++g) {
                        const float e = ee[j][g], dx = dxs[j][g];
                        float Gv = pv[C];  // -s
#pragma unroll
                        for (int c = 0; c < C; ++c) Gv = fmaf(pv[c], col[g][c], Gv);
                        const float ge = Gv * e;
                        R0[g] += ge;
                        const float t1 = ge * dx;
                        R1[g] += t1;
                        R2[g] = fmaf(t1, dx, R2[g]);
#pragma unroll
                        for (int c = 0; c < C; ++c) RC[g][c] = fmaf(e, pv[c], RC[g][c]);
                    }
                }
            }
            // the tile row is complete
#pragma unroll
            for (int g = 0; g < G; ++g) {
                M[g][0] += R0[g];
                M[g][1] += R1[g];
                M[g][3] += R2[g];
                M[g][2] = fmaf(dy[g], R0[g], M[g][2]);
                M[g][4] = fmaf(dy[g], R1[g], M[g][4]);
                M[g][5] = fmaf(dy[g] * dy[g], R0[g], M[g][5]);
#pragma unroll
                for (int c = 0; c < C; ++c) CG[g][c] += RC[g][c];
            }
        }
        if (k + 1 < chunks) {
            float4* nxt = sh + ((k + 1) & 1) * E;
#pragma unroll
            for (int i = 0; i < PRE; ++i) {
                const int e = i * kThreads + tid;
                if (e < E) nxt[e] = pre[i];
            }
            if (tid <= RPC) ysh[(k + 1) & 1][tid] = ypre;
        }
        __syncthreads();
    }
    bwd_store<C, G>(a, b, t, slot, M, CG);
}

// General grid: the tile is a flat pixel range (multiple of 256); x and y come with the
// pixel record.  Sums are flushed into the totals once per 128-pixel chunk.
template <int C, int G>
__global__ __launch_bounds__(kThreads) void k_bwd_gen(const BwdArgs a) {
    constexpr int CP = pix_stride_gen(C), CP4 = CP / 4;
    constexpr int kPixChunk = pix_chunk(C);
    __shared__ float4 sh[2 * kPixChunk * CP4];
    IGS_GATE(a);
    const int b = blockIdx.z, t = blockIdx.y;
    int n[G];
#pragma unroll
    for (int g = 0; g < G; ++g) n[g] = (blockIdx.x * G + g) * kThreads + threadIdx.x;
    float px[G], py[G], A[G], B2[G], D[G], col[G][C];
    bwd_load_gaussians<C, G>(a, b, n, px, py, A, B2, D, col);
    float M[G][6], CG[G][C], R[G][6], RC[G][C];
#pragma unroll
    for (int g = 0; g < G; ++g) {
#pragma unroll
        for (int f = 0; f < 6; ++f) M[g][f] = R[g][f] = 0.0f;
#pragma unroll
        for (int c = 0; c < C; ++c) CG[g][c] = RC[g][c] = 0.0f;
    }
    const int p0 = t * a.per_tile, p1 = min(a.HWp, p0 + a.per_tile);
    const float4* src = reinterpret_cast<const float4*>(a.pixrec + ((size_t)b * a.HWp + p0) * CP);
    int seen = 0;
    stream_records_lds<CP4, kPixChunk>(src, p1 - p0, sh, [&](const float4* r) {
        float pv[CP];
#pragma unroll
        for (int q4 = 0; q4 < CP4; ++q4) {
            const float4 tq = r[q4];
            pv[4 * q4] = tq.x;
            pv[4 * q4 + 1] = tq.y;
            pv[4 * q4 + 2] = tq.z;
            pv[4 * q4 + 3] = tq.w;
        }
        float dxs[G], dys[G], ee[G];
#pragma unroll
        for (int g = 0; g < G; ++g) {
            const float dx = pv[0] - px[g];
            const float dy = pv[1] - py[g];
            float tt = A[g] * dx;
            tt = fmaf(B2[g], dy, tt);
            const float v = D[g] * dy;
            float q = tt * dx;
            ee[g] = fmaf(v, dy, q);
            dxs[g] = dx;
            dys[g] = dy;
        }
#pragma unroll
        for (int g = 0; g < G; ++g) ee[g] = hw_exp2(ee[g]);
#pragma unroll
        for (int g = 0; g < G; ++g) {
            const float e = ee[g], dx = dxs[g], dy = dys[g];
            float Gv = pv[2 + C];  // -s
#pragma unroll
            for (int c = 0; c < C; ++c) Gv = fmaf(pv[2 + c], col[g][c], Gv);
            const float ge = Gv * e;
            R[g][0] += ge;
            const float t1 = ge * dx, t2 = ge * dy;
            R[g][1] += t1;
            R[g][2] += t2;
            R[g][3] = fmaf(t1, dx, R[g][3]);
            R[g][4] = fmaf(t1, dy, R[g][4]);
            R[g][5] = fmaf(t2, dy, R[g][5]);
#pragma unroll
            for (int c = 0; c < C; ++c) RC[g][c] = fmaf(e, pv[2 + c], RC[g][c]);
        }
        if ((++seen & (kPixChunk - 1)) == 0) {  // two-level summation
#pragma unroll
            for (int g = 0; g < G; ++g) {
#pragma unroll
                for (int f = 0; f < 6; ++f) {
                    M[g][f] += R[g][f];
                    R[g][f] = 0.0f;
                }
#pragma unroll
                for (int c = 0; c < C; ++c) {
                    CG[g][c] += RC[g][c];
                    RC[g][c] = 0.0f;
                }
            }
        }
    });
#pragma unroll
    for (int g = 0; g < G; ++g) {
#pragma unroll
        for (int f = 0; f < 6; ++f) M[g][f] += R[g][f];
#pragma unroll
        for (int c = 0; c < C; ++c) CG[g][c] += RC[g][c];
    }
    bwd_store<C, G>(a, b, t, n, M, CG);
}

// Fixed-order sum over the T tile partials of NV consecutive fields for one Gaussian, spread
// over the kFinT "t-lanes" of a workgroup laid out as kFinT t-lanes x kFinN Gaussians: t-lane k
// adds tiles k, k+kFinT, ... in order, the lane sums are then added in order by every thread (so
// all t-lanes of a Gaussian hold the same, run-to-run identical value).  `red` is
// [NV][kFinT][kFinN+1] floats of LDS.  Must be called by all 256 threads.  (8 x 32: with fewer
// t-lanes the consecutive Gaussians of a wave read neighbouring columns of a tile's partials,
// with more the sequential part of a sum over hundreds of tiles gets shorter.)
#ifndef IGS_FIN_T
#define IGS_FIN_T 8
#endif
constexpr int kFinT = IGS_FIN_T, kFinN = 256 / IGS_FIN_T;
constexpr int kFinColours = 8;  // colour channels summed per pass (>= 6: the LDS array also serves the moments)

// `part` is the image's partial array [T][NF][N]; the Gaussian's column in tile t is
// slots[t * Np + n] when a slot table is given (negative: the tile holds nothing for it), else n.
// Only the first `nv` (<= NV) of the fields are read.
template <int NV>
__device__ __forceinline__ void tile_sum(const float* __restrict__ part, const int* __restrict__ slots,
                                         int Np, int n, int T, int NF, int N, int f0, bool valid,
                                         float (&out)[NV], float* red, int nv = NV) {
    const int tl = threadIdx.x / kFinN, nl = threadIdx.x % kFinN;
    float acc[NV];
#pragma unroll
    for (int v = 0; v < NV; ++v) acc[v] = 0.0f;
    if (valid)
        for (int t = tl; t < T; t += kFinT) {
            const int col = slots ? slots[(size_t)t * Np + n] : n;
            if (col >= 0) {
#pragma unroll
                for (int v = 0; v < NV; ++v)
                    if (v < nv) acc[v] += part[((size_t)t * NF + f0 + v) * N + col];
            }
        }
    __syncthreads();  // protects `red` against the previous call's readers
#pragma unroll
    for (int v = 0; v < NV; ++v) red[(v * kFinT + tl) * (kFinN + 1) + nl] = acc[v];
    __syncthreads();
#pragma unroll
    for (int v = 0; v < NV; ++v) {
        float s = 0.0f;
#pragma unroll
        for (int k = 0; k < kFinT; ++k) s += red[(v * kFinT + k) * (kFinN + 1) + nl];
        out[v] = s;
    }
}

// Finalize: 16 threads per Gaussian; sums the T tile partials in a fixed order and applies
//   d alpha = M0, d color_c = alpha CG_c, d px = alpha (A Mx + B My), d py = alpha (B Mx + D My),
//   dA = -1/2 alpha Mxx, dB = -alpha Mxy, dD = -1/2 alpha Myy,
// and (function level) the chain rule through A = c^2 i0 + s^2 i1, B = c s (i0 - i1),
// D = s^2 i0 + c^2 i1, i_k = 1/(s_k^2 + eps).
template <bool kScaleRot>
__global__ __launch_bounds__(kThreads) void k_bwd_finalize(
    const float* __restrict__ partial, int T_in, const int* __restrict__ flag, int T_alt,
    const int* __restrict__ slots_in, int Np, const float* __restrict__ p0,
    const float* __restrict__ p1, const float* __restrict__ p2, const float* __restrict__ alphas,
    int N, int C, float eps, float* __restrict__ g_pos, float* __restrict__ g0,
    float* __restrict__ g1, float* __restrict__ g2, float* __restrict__ g_alpha,
    float* __restrict__ g_col) {
    __shared__ float red[kFinColours * kFinT * (kFinN + 1)];
    const int n = blockIdx.x * kFinN + threadIdx.x % kFinN;
    const int b = blockIdx.y;
    const bool valid = n < N;
    const bool writer = valid && threadIdx.x < kFinN;  // t-lane 0 writes the results
    // AUTO grid mode: T_in belongs to the separable plan, T_alt to the general one
    const int T = (flag != nullptr && *flag == 0) ? T_alt : T_in;
    const int NF = 6 + C;
    const size_t i = (size_t)b * N + min(n, N - 1);
    const float* part = partial + (size_t)b * T * NF * N;
    // the slot table belongs to the separable variant
    const int* slots = (slots_in != nullptr && !(flag != nullptr && *flag == 0))
                           ? slots_in + (size_t)b * T * Np : nullptr;
    const int nn = min(n, N - 1);
    float M[6];
    tile_sum<6>(part, slots, Np, nn, T, NF, N, 0, valid, M, red);
    const double al = alphas[i];
    // O(BN) epilogue in fp64: the chain rule multiplies sums by 1/s^3-sized factors
    double A, Bc, D, cs = 0., sn = 0., i0 = 0., i1 = 0., s0 = 0., s1 = 0.;
    if (kScaleRot) {
        s0 = p0[2 * i];
        s1 = p0[2 * i + 1];
        sincos((double)p1[i], &sn, &cs);
        i0 = 1.0 / (s0 * s0 + (double)eps);
        i1 = 1.0 / (s1 * s1 + (double)eps);
        A = cs * cs * i0 + sn * sn * i1;
        Bc = cs * sn * (i0 - i1);
        D = sn * sn * i0 + cs * cs * i1;
    } else {
        A = p0[i];
        Bc = p1[i];
        D = p2[i];
    }
    if (g_alpha && writer) g_alpha[i] = M[0];
    if (g_pos && writer) {
        g_pos[2 * i] = (float)(al * (A * M[1] + Bc * M[2]));
        g_pos[2 * i + 1] = (float)(al * (Bc * M[1] + D * M[2]));
    }
    const double gA = -0.5 * al * M[3], gB = -al * M[4], gD = -0.5 * al * M[5];
    if (kScaleRot) {
        if (g0 && writer) {  // scales [B,N,2]
            const double gi0 = gA * cs * cs + gB * cs * sn + gD * sn * sn;
            const double gi1 = gA * sn * sn - gB * cs * sn + gD * cs * cs;
            g0[2 * i] = (float)(gi0 * (-2.0 * s0 * i0 * i0));
            g0[2 * i + 1] = (float)(gi1 * (-2.0 * s1 * i1 * i1));
        }
        if (g1 && writer) g1[i] = (float)((gD - gA) * 2.0 * Bc + gB * (cs * cs - sn * sn) * (i0 - i1));
    } else {
        if (g0 && writer) g0[i] = (float)gA;
        if (g1 && writer) g1[i] = (float)gB;
        if (g2 && writer) g2[i] = (float)gD;
    }
    if (g_col) {  // kernel-argument uniform, so the barriers inside tile_sum are safe
        for (int c0 = 0; c0 < C; c0 += kFinColours) {  // colour sums, kFinColours channels per pass
            float sc[kFinColours];
            const int nc = min(kFinColours, C - c0);
            tile_sum<kFinColours>(part, slots, Np, nn, T, NF, N, 6 + c0, valid, sc, red, nc);
            if (writer)
#pragma unroll
                for (int c = 0; c < kFinColours; ++c)
                    if (c < nc) g_col[i * C + c0 + c] = (float)al * sc[c];
        }
    }
}

// Finalize for the fused module head: d gs_feature [B][N][6+C] from the tile partials, with
// alpha = 1, d log_s_k = d s_k * exp(log_s_k) and a zero gradient for the unused opacity logit.
__global__ __launch_bounds__(kThreads) void k_bwd_finalize_feature(
    const float* __restrict__ partial, int T_in, const int* __restrict__ flag, int T_alt,
    const int* __restrict__ slots_in, int Np, const float* __restrict__ feat, int N, int C, int Cp,
    float eps, float* __restrict__ g_feat) {
    __shared__ float red[kFinColours * kFinT * (kFinN + 1)];
    const int n = blockIdx.x * kFinN + threadIdx.x % kFinN;
    const int b = blockIdx.y;
    const bool valid = n < N;
    const bool writer = valid && threadIdx.x < kFinN;
    const int T = (flag != nullptr && *flag == 0) ? T_alt : T_in;
    const int NF = 6 + Cp;
    const size_t i = (size_t)b * N + min(n, N - 1);
    const float* part = partial + (size_t)b * T * NF * N;
    const int* slots = (slots_in != nullptr && !(flag != nullptr && *flag == 0))
                           ? slots_in + (size_t)b * T * Np : nullptr;
    const int nn = min(n, N - 1);
    float M[6];
    tile_sum<6>(part, slots, Np, nn, T, NF, N, 0, valid, M, red);
    const float* f = feat + i * (6 + C);
    const double e0 = (double)expf(f[2]), e1 = (double)expf(f[3]);
    const double s0 = e0 + (double)eps, s1 = e1 + (double)eps;
    double sn, cs;
    sincos((double)f[4], &sn, &cs);
    const double i0 = 1.0 / (s0 * s0 + (double)eps), i1 = 1.0 / (s1 * s1 + (double)eps);
    const double A = cs * cs * i0 + sn * sn * i1;
    const double Bc = cs * sn * (i0 - i1);
    const double D = sn * sn * i0 + cs * cs * i1;
    const double gA = -0.5 * M[3], gB = -(double)M[4], gD = -0.5 * M[5];
    const double gi0 = gA * cs * cs + gB * cs * sn + gD * sn * sn;
    const double gi1 = gA * sn * sn - gB * cs * sn + gD * cs * cs;
    float* g = g_feat + i * (6 + C);
    if (writer) {
        g[0] = (float)(A * M[1] + Bc * M[2]);
        g[1] = (float)(Bc * M[1] + D * M[2]);
        g[2] = (float)(gi0 * (-2.0 * s0 * i0 * i0) * e0);
        g[3] = (float)(gi1 * (-2.0 * s1 * i1 * i1) * e1);
        g[4] = (float)((gD - gA) * 2.0 * Bc + gB * (cs * cs - sn * sn) * (i0 - i1));
        g[5] = 0.0f;
    }
    for (int c0 = 0; c0 < C; c0 += kFinColours) {
        float sc[kFinColours];
        const int nc = min(kFinColours, C - c0);
        tile_sum<kFinColours>(part, slots, Np, nn, T, NF, N, 6 + c0, valid, sc, red, nc);
        if (writer)
#pragma unroll
            for (int c = 0; c < kFinColours; ++c)
                if (c < nc) g[6 + c0 + c] = sc[c];
    }
}

// ----------------------------------------------------------------------------- grid grads
// Optional: d L / d x(pixel), d L / d y(pixel) = -sum_n G_n w_n (A dx + B dy), (B dx + D dy).
// Pixel-major like the forward (lane = P pixels, Gaussian record wave-uniform); the per-pixel
// g^, s are rebuilt from out/den/grad_out in the prologue of the same kernel.  With
// t1 = A'dx + (B2'/2) dy and t2 = (B2'/2) dx + D'dy the exponent is q' = dx t1 + dy t2, and
// the sums of G w t1, G w t2 are scaled by -1/k (k = -0.5 log2 e) at the end.
struct GridGradArgs {
    const float* packed;
    const float* x;
    const float* y;
    long sxb, sxh, sxw, syb, syh, syw;
    const float* out;
    const float* den;
    const float* gout;
    int Np, H, W, tiles_per_img, total_tiles;
    float eps;
    float* gx;  // [B][H*W]
    float* gy;
};

template <int C, int P>
__global__ __launch_bounds__(kThreads) void k_bwd_grid(const GridGradArgs a) {
    constexpr int RS = rec_stride_of(C), R4 = RS / 4;
    __shared__ float4 sh[2 * kGaussChunk * R4];
    const int tile = xcd_contiguous(blockIdx.x, a.total_tiles);
    if (tile >= a.total_tiles) return;  // workgroup-uniform
    const int b = tile / a.tiles_per_img;
    const int tl = tile - b * a.tiles_per_img;
    const int HW = a.H * a.W;
    float xv[P], yv[P], gh[P][C], negs[P], sx[P], sy[P];
    int pix[P];
#pragma unroll
    for (int j = 0; j < P; ++j) {
        pix[j] = tl * (kThreads * P) + j * kThreads + (int)threadIdx.x;
        const int pc = min(pix[j], HW - 1);
        const int h = pc / a.W, w = pc - h * a.W;
        xv[j] = a.x[b * a.sxb + h * a.sxh + w * a.sxw];
        yv[j] = a.y[b * a.syb + h * a.syh + w * a.syw];
        const float inv = 1.0f / (a.den[(size_t)b * HW + pc] + a.eps);
        float s = 0.0f;
#pragma unroll
        for (int c = 0; c < C; ++c) {
            gh[j][c] = a.gout[((size_t)b * C + c) * HW + pc] * inv;
            s = fmaf(gh[j][c], a.out[((size_t)b * C + c) * HW + pc], s);
        }
        negs[j] = -s;
        sx[j] = sy[j] = 0.0f;
    }
    const float4* src = reinterpret_cast<const float4*>(a.packed + (size_t)b * a.Np * RS);
    stream_records_lds<R4, kGaussChunk>(src, a.Np, sh, [&](const float4* r) {
        const GRec<C> g = lds_grec<C>(r);
        const float hb = 0.5f * g.B2;
        // phases: exponents, transcendentals back to back, accumulation
        float t1[P], t2[P], e[P];
#pragma unroll
        for (int j = 0; j < P; ++j) {
            const float dx = xv[j] - g.px;
            const float dy = yv[j] - g.py;
            t1[j] = fmaf(g.A, dx, hb * dy);
            t2[j] = fmaf(g.D, dy, hb * dx);
            e[j] = fmaf(dx, t1[j], dy * t2[j]);
        }
#pragma unroll
        for (int j = 0; j < P; ++j) e[j] = hw_exp2(e[j]);
#pragma unroll
        for (int j = 0; j < P; ++j) {
            float Gv = negs[j] * g.al;  // alpha (<g^, c> - s)
#pragma unroll
            for (int c = 0; c < C; ++c) Gv = fmaf(gh[j][c], g.ac[c], Gv);
            const float Gw = Gv * e[j];
            sx[j] = fmaf(Gw, t1[j], sx[j]);
            sy[j] = fmaf(Gw, t2[j], sy[j]);
        }
    });
    constexpr float kScale = -1.0f / kNegHalfLog2e;  // A dx + B dy = t1 / k, and the leading minus
#pragma unroll
    for (int j = 0; j < P; ++j)
        if (pix[j] < HW) {
            a.gx[(size_t)b * HW + pix[j]] = kScale * sx[j];
            a.gy[(size_t)b * HW + pix[j]] = kScale * sy[j];
        }
}

// ----------------------------------------------------------------------------- grid class
// flag = 1 iff x does not depend on the row and y does not depend on the column (bitwise).
__global__ void k_flag_set(int* flag, int v) {
    if (threadIdx.x == 0 && blockIdx.x == 0) *flag = v;
}

__global__ __launch_bounds__(kThreads) void k_grid_classify(const float* __restrict__ x,
                                                            const float* __restrict__ y, long sxb,
                                                            long sxh, long sxw, long syb, long syh,
                                                            long syw, int H, int W,
                                                            int* __restrict__ flag) {
    const int p = blockIdx.x * kThreads + threadIdx.x;
    const int b = blockIdx.y;
    if (p >= H * W) return;
    const int h = p / W, w = p - h * W;
    const float xv = x[b * sxb + h * sxh + w * sxw], x0 = x[b * sxb + w * sxw];
    const float yv = y[b * syb + h * syh + w * syw], y0 = y[b * syb + h * syh];
    // every writer stores the same value, so the race between them is benign
    if (__float_as_uint(xv) != __float_as_uint(x0) || __float_as_uint(yv) != __float_as_uint(y0))
        *flag = 0;
}

// ----------------------------------------------------------------------------- host side
int g_cached_cus = 0;

int device_cus() {
    if (g_cached_cus > 0) return g_cached_cus;
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) return 0;
    int cus = 0;
    if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess) return 0;
    g_cached_cus = cus;
    return cus;
}

inline int ceil_div(long a, long b) { return (int)((a + b - 1) / b); }

bool shape_ok(int B, int N, int H, int W) {
    if (B <= 0 || N <= 0 || H <= 0 || W <= 0) return false;
    if (B > 65535) return false;
    if ((long)H * W > (1L << 28) || (long)B * N > (1L << 28)) return false;
    return true;
}

struct FwdGeometry {
    int wx, tiles_x, tiles_y, total_tiles;
};

FwdGeometry fwd_geometry(int B, int H, int W, int C, bool sep) {
    FwdGeometry g;
    const int kFwdSepP = fwd_sep_p(C);
    if (sep) {
        // choose the wave arrangement (wx waves along the columns) that wastes the fewest lanes;
        // on a tie the squarest tile (fewest Gaussians reach it)
        long best = -1;
        g.wx = 1;
        for (int wx = 1; wx <= 4; wx <<= 1) {
            const long cols = (long)ceil_div(W, 64 * wx) * 64 * wx;
            const long rows = (long)ceil_div(H, kFwdSepP * (4 / wx)) * kFwdSepP * (4 / wx);
            const long area = cols * rows;
            if (best < 0 || area < best) {
                best = area;
                g.wx = wx;
            }
        }
        g.tiles_x = ceil_div(W, 64 * g.wx);
        g.tiles_y = ceil_div(H, kFwdSepP * (4 / g.wx));
    } else {
        g.wx = 4;
        g.tiles_x = ceil_div((long)H * W, kThreads * fwd_gen_p(C));
        g.tiles_y = 1;
    }
    g.total_tiles = B * g.tiles_x * g.tiles_y;
    return g;
}

// Tile lists of one launch: counts [B][tiles] (padded to 4 ints) then lists [B][tiles][Np].
inline size_t bins_bytes(int B, int tiles, int Np) {
    return ((((size_t)B * tiles + 3) & ~(size_t)3) + (size_t)B * tiles * Np) * sizeof(int);
}
inline size_t align16(size_t v) { return (v + 15) & ~(size_t)15; }

// Plan of one kernel variant (grid_mode is GENERAL or SEPARABLE here).
int plan_one(int B, int N, int H, int W, int C, int grid_mode, igs_gs2d_plan_t* p) {
    if (!p) return IGS_ERR_NULL_POINTER;
    if (!shape_ok(B, N, H, W)) return IGS_ERR_BAD_SHAPE;
    if (C < 1 || C > IGS_MAX_CHANNELS) return IGS_ERR_BAD_CHANNELS;
    if (grid_mode != IGS_GRID_GENERAL && grid_mode != IGS_GRID_SEPARABLE) return IGS_ERR_BAD_MODE;
    const bool sep = grid_mode == IGS_GRID_SEPARABLE;
    int cus = device_cus();
    if (cus <= 0) cus = 256;
    const long target_waves = (long)cus * 4 * IGS_FWD_WAVES;  // forward: waves per SIMD wanted
    p->B = B; p->N = N; p->H = H; p->W = W; p->C = C;
    p->rec_stride = rec_stride_of(C);
    p->n_padded = (N + 3) & ~3;
    p->w_padded = sep ? (W + 7) & ~7 : W;
    p->hw_padded = (H * W + 3) & ~3;
    const FwdGeometry fg = fwd_geometry(B, H, W, C, sep);
    long S = (target_waves + (long)fg.total_tiles * 4 - 1) / ((long)fg.total_tiles * 4);
    const long maxS = N / 64 > 0 ? N / 64 : 1;  // keep >= 64 Gaussians per split
    if (S > maxS) S = maxS;
    if (S > 64) S = 64;
    if (S < 1) S = 1;
    // Gaussians per split: a multiple of 4; drop splits that would be empty
    const int nps = (ceil_div(p->n_padded, S) + 3) & ~3;
    S = ceil_div(p->n_padded, nps);
    p->fwd_split = (int)S;
    p->fwd_n_per_split = nps;
    const long groups = (long)B * ceil_div(N, kThreads * (sep ? kBwdG : bwd_gen_g(C))) * 4;  // waves per tile
    long T = ((long)cus * 4 * IGS_BWD_WAVES + groups - 1) / groups;     // backward: waves per SIMD wanted
    p->bwd_tiles_x = sep ? ceil_div(p->w_padded, kBwdTileW) : 1;
    if (sep) {
        T = (T + p->bwd_tiles_x - 1) / p->bwd_tiles_x;                  // row bands
        // small tiles keep the tile lists short when the Gaussians are small (a tile is skipped
        // by every Gaussian whose reach box misses it): at most kBwdMaxRows rows per tile
        const long bands = ceil_div(H, kBwdMaxRows);
        if (T < bands) T = bands;
    }
    // (tiles of fewer than kBwdMinRows rows cost more in partial sums than they gain in fill)
    const long maxT = sep ? ceil_div(H, kBwdMinRows) : ceil_div(p->hw_padded, 256);
    if (T > maxT) T = maxT;
    if (T < 1) T = 1;
    if (sep) {
        p->bwd_per_tile = ceil_div(H, T);
    } else {
        p->bwd_per_tile = (ceil_div(p->hw_padded, T) + 255) & ~255;
    }
    T = (long)ceil_div(sep ? H : p->hw_padded, p->bwd_per_tile) * p->bwd_tiles_x;
    p->bwd_tiles = (int)T;
    p->fwd_tiles = sep ? fg.tiles_x * fg.tiles_y : 0;
    p->pix_stride = sep ? pix_stride_sep(C) : pix_stride_gen(C);
    // records, then one reach box (4 floats) per record
    p->packed_bytes = (uint64_t)B * p->n_padded * (p->rec_stride + 4) * sizeof(float);
    p->fwd_ws_bytes = S > 1 ? (uint64_t)S * B * (C + 1) * H * W * sizeof(float) : 0;
    p->pix_bytes = sep ? ((uint64_t)B * H * p->w_padded * p->pix_stride + (uint64_t)B * p->w_padded) * sizeof(float)
                       : (uint64_t)B * p->hw_padded * p->pix_stride * sizeof(float);
    if (sep) {  // the tile lists of each launch follow its other scratch
        p->fwd_ws_bytes = align16(p->fwd_ws_bytes) + bins_bytes(B, p->fwd_tiles, p->n_padded);
        p->pix_bytes = align16(p->pix_bytes) + bins_bytes(B, p->bwd_tiles, p->n_padded);
    }
    p->partial_bytes = (uint64_t)B * T * (6 + C) * N * sizeof(float);
    if (sep)  // the slot tables [B][T][Np] (Gaussian -> position in the tile's list) follow
        p->partial_bytes = align16(p->partial_bytes) + (uint64_t)B * T * p->n_padded * sizeof(int);
    return IGS_OK;
}

// The slot tables of the separable backward inside the partial buffer.
inline int* slots_at(float* partial, int B, int T, int NF, int N) {
    return reinterpret_cast<int*>(reinterpret_cast<char*>(partial) +
                                  align16((size_t)B * T * NF * N * sizeof(float)));
}

// Where the tile lists of a separable launch live inside its workspace.
struct BinPlace {
    int* counts;
    int* lists;
};
inline BinPlace bins_at(void* ws, size_t scratch_bytes, int B, int tiles) {
    char* base = static_cast<char*>(ws) + align16(scratch_bytes);
    BinPlace bp;
    bp.counts = reinterpret_cast<int*>(base);
    bp.lists = bp.counts + (((size_t)B * tiles + 3) & ~(size_t)3);
    return bp;
}

inline const float4* boxes_of(const float* packed, int B, int Np, int RS) {
    return reinterpret_cast<const float4*>(packed + (size_t)B * Np * RS);
}

// IGS_NO_CULL=1 in the environment makes every reach box unbounded (nothing is skipped): the
// reference point for checking that culling changes no bit.  Read at every pack call.
inline int culling_enabled() {
    const char* e = getenv("IGS_NO_CULL");
    return !(e && e[0] == '1');
}

// Public plan: AUTO reports the separable variant's geometry with the workspace sizes of
// whichever variant needs more.
int make_plan(int B, int N, int H, int W, int C, int grid_mode, igs_gs2d_plan_t* p) {
    if (grid_mode != IGS_GRID_AUTO) return plan_one(B, N, H, W, C, grid_mode, p);
    igs_gs2d_plan_t g;
    int rc = plan_one(B, N, H, W, C, IGS_GRID_SEPARABLE, p);
    if (rc) return rc;
    rc = plan_one(B, N, H, W, C, IGS_GRID_GENERAL, &g);
    if (rc) return rc;
    if (g.fwd_ws_bytes > p->fwd_ws_bytes) p->fwd_ws_bytes = g.fwd_ws_bytes;
    if (g.pix_bytes > p->pix_bytes) p->pix_bytes = g.pix_bytes;
    if (g.partial_bytes > p->partial_bytes) p->partial_bytes = g.partial_bytes;
    return IGS_OK;
}

int launch_bin(const BinArgs& a, int B, hipStream_t st) {
    hipLaunchKernelGGL(k_bin, dim3(a.tiles_x * a.tiles_y, B), dim3(kBinThreads), 0, st, a);
    const hipError_t e = hipGetLastError();
    return e == hipSuccess ? IGS_OK : (int)e;
}

inline int launch_status() {
    const hipError_t e = hipGetLastError();
    return e == hipSuccess ? IGS_OK : (int)e;
}

bool channels_compiled(int C) { return C == 1 || C == 2 || C == 3 || C == 4 || C == 8 || C == 16; }

// Channel counts with a compiled specialisation; other C <= 16 are rejected by the ABI
// (the host wrapper zero-pads colours / grad_out up to the next one, which is exact).
#define IGS_DISPATCH_C(C, CALL)                          \
    switch (C) {                                         \
        case 1: { constexpr int kC = 1; CALL; } break;   \
        case 2: { constexpr int kC = 2; CALL; } break;   \
        case 3: { constexpr int kC = 3; CALL; } break;   \
        case 4: { constexpr int kC = 4; CALL; } break;   \
        case 8: { constexpr int kC = 8; CALL; } break;   \
        case 16: { constexpr int kC = 16; CALL; } break; \
        default: return IGS_ERR_BAD_CHANNELS;            \
    }

// The variants a grid mode runs: {variant mode, flag value it is gated on}; AUTO runs both.
struct Variant {
    int mode;
    const int* flag;
    int want;
};

int variants_of(int grid_mode, const int32_t* grid_flag, Variant (&v)[2]) {
    if (grid_mode == IGS_GRID_AUTO) {
        v[0] = {IGS_GRID_SEPARABLE, grid_flag, 1};
        v[1] = {IGS_GRID_GENERAL, grid_flag, 0};
        return 2;
    }
    v[0] = {grid_mode, nullptr, 0};
    return 1;
}

// Fused mean-squared-error upstream gradient of the fit step (all null/zero: plain backward).
struct MseArgs {
    const float* target = nullptr;  // [B,C,H,W]
    float gscale = 0.0f;            // 2 / (number of real elements)
    float* loss_part = nullptr;     // one float per prologue workgroup
    float loss_scale = 0.0f;        // 1 / (number of real elements)
    float* loss = nullptr;          // 1 float
};

template <int C>
int launch_forward(const FwdArgs& a, bool sep, hipStream_t st) {
    const int blocks = ((a.total_tiles + 7) / 8) * 8;
    const dim3 grid(blocks, a.S, 1);
    if (sep)
        hipLaunchKernelGGL((k_fwd_sep<C, fwd_sep_p(C)>), grid, dim3(kThreads), 0, st, a);
    else
        hipLaunchKernelGGL((k_fwd_gen<C, fwd_gen_p(C)>), grid, dim3(kThreads), 0, st, a);
    return launch_status();
}

template <int C>
int launch_bwd_prologue(const BwdArgs& a, int B, bool sep, const float* out, const float* den,
                        const float* gout, const MseArgs& mse, const float* x, const float* y,
                        const int64_t* gs, float eps, float* pixrec, hipStream_t st) {
    const int padded = sep ? a.H * a.Wp : a.HWp;
    const dim3 pgrid(ceil_div(padded, kThreads), B, 1);
    if (sep)
        hipLaunchKernelGGL((k_bwd_pix<C, true>), pgrid, dim3(kThreads), 0, st, out, den, gout,
                           mse.target, mse.gscale, mse.loss_part, x, y,
                           gs[0], gs[1], gs[2], gs[3], gs[4], gs[5], B, a.H, a.W, a.Wp, a.HWp, eps,
                           pixrec, a.flag, a.want);
    else
        hipLaunchKernelGGL((k_bwd_pix<C, false>), pgrid, dim3(kThreads), 0, st, out, den, gout,
                           mse.target, mse.gscale, mse.loss_part, x, y,
                           gs[0], gs[1], gs[2], gs[3], gs[4], gs[5], B, a.H, a.W, a.Wp, a.HWp, eps,
                           pixrec, a.flag, a.want);
    int rc = launch_status();
    if (rc || !mse.loss_part) return rc;
    hipLaunchKernelGGL(k_loss_sum, dim3(1), dim3(kThreads), 0, st, mse.loss_part, (int)pgrid.x * B,
                       mse.loss_scale, mse.loss, a.flag, a.want);
    return launch_status();
}

template <int C>
int launch_bwd_reduce(const BwdArgs& a, int B, bool sep, hipStream_t st) {
    if (sep) {
        // every list position up to Np is visited: listed Gaussians compute, the others store zeros
        const dim3 grid(a.T, ceil_div(a.Np, kThreads * kBwdG), B);
        hipLaunchKernelGGL((k_bwd_sep<C, kBwdG>), grid, dim3(kThreads), 0, st, a);
    } else {
        const dim3 grid(ceil_div(a.N, kThreads * bwd_gen_g(C)), a.T, B);
        hipLaunchKernelGGL((k_bwd_gen<C, bwd_gen_g(C)>), grid, dim3(kThreads), 0, st, a);
    }
    return launch_status();
}

int bwd_args(BwdArgs& a, const Variant& v, const float* packed, const float* colors, const float* y,
             const int64_t gs[6], int B, int N, int H, int W, int C, float* pix_ws, float* partial) {
    igs_gs2d_plan_t plan;
    const int rc = plan_one(B, N, H, W, C, v.mode, &plan);
    if (rc) return rc;
    const bool sep = v.mode == IGS_GRID_SEPARABLE;
    a.packed = packed; a.colors = colors; a.pixrec = pix_ws;
    a.xs = sep ? pix_ws + (size_t)B * H * plan.w_padded * plan.pix_stride : nullptr;
    a.y = y;
    a.syb = gs[3]; a.syh = gs[4];
    a.N = N; a.Np = plan.n_padded; a.H = H; a.W = W; a.Wp = plan.w_padded; a.HWp = plan.hw_padded;
    a.T = plan.bwd_tiles;
    a.tiles_x = plan.bwd_tiles_x;
    a.per_tile = plan.bwd_per_tile;
    a.counts = nullptr; a.lists = nullptr;
    if (sep && pix_ws) {
        const size_t scratch = ((size_t)B * H * plan.w_padded * plan.pix_stride + (size_t)B * plan.w_padded) * sizeof(float);
        const BinPlace bp = bins_at(pix_ws, scratch, B, plan.bwd_tiles);
        a.counts = bp.counts; a.lists = bp.lists;
    }
    a.partial = partial;
    a.flag = v.flag; a.want = v.want;
    return IGS_OK;
}

int mode_ok(int grid_mode, const int32_t* grid_flag) {
    if (grid_mode != IGS_GRID_GENERAL && grid_mode != IGS_GRID_SEPARABLE && grid_mode != IGS_GRID_AUTO)
        return IGS_ERR_BAD_MODE;
    if (grid_mode == IGS_GRID_AUTO && !grid_flag) return IGS_ERR_NULL_POINTER;
    return IGS_OK;
}

}  // namespace

// ============================================================================= C ABI
extern "C" {

int igs_abi_version(void) { return IGS_ABI_VERSION; }

const char* igs_status_string(int status) {
    switch (status) {
        case IGS_OK: return "ok";
        case IGS_ERR_NULL_POINTER: return "null pointer argument";
        case IGS_ERR_BAD_SHAPE: return "bad shape (dimension <= 0 or too large)";
        case IGS_ERR_BAD_CHANNELS: return "unsupported channel count (compiled: 1, 2, 3, 4, 8, 16)";
        case IGS_ERR_WORKSPACE: return "workspace smaller than igs_gs2d_plan requires";
        case IGS_ERR_BAD_MODE: return "unknown grid mode";
        case IGS_ERR_NO_DEVICE: return "no usable HIP device";
        case IGS_ERR_ALIGNMENT: return "buffer not 16-byte aligned";
        default: break;
    }
    if (status > 0) return hipGetErrorString((hipError_t)status);
    return "unknown igs status";
}

int igs_gs2d_plan(int B, int N, int H, int W, int C, int grid_mode, igs_gs2d_plan_t* plan) {
    const int rc = make_plan(B, N, H, W, C, grid_mode, plan);
    if (rc) return rc;
    return channels_compiled(C) ? IGS_OK : IGS_ERR_BAD_CHANNELS;
}

int igs_gs2d_grid_classify(const float* x, const float* y, const int64_t grid_strides[6], int B,
                           int H, int W, int32_t* grid_flag, igs_stream_t stream) {
    if (!x || !y || !grid_strides || !grid_flag) return IGS_ERR_NULL_POINTER;
    if (!shape_ok(B, 1, H, W)) return IGS_ERR_BAD_SHAPE;
    hipStream_t st = (hipStream_t)stream;
    hipLaunchKernelGGL(k_flag_set, dim3(1), dim3(64), 0, st, grid_flag, 1);
    hipLaunchKernelGGL(k_grid_classify, dim3(ceil_div((long)H * W, kThreads), B), dim3(kThreads), 0, st,
                       x, y, grid_strides[0], grid_strides[1], grid_strides[2], grid_strides[3],
                       grid_strides[4], grid_strides[5], H, W, grid_flag);
    return launch_status();
}

int igs_gs2d_pack_covinv(const float* position, const float* cov_inv_00, const float* cov_inv_01,
                         const float* cov_inv_11, const float* alphas, const float* colors, int B,
                         int N, int C, float* packed, igs_stream_t stream) {
    if (!position || !cov_inv_00 || !cov_inv_01 || !cov_inv_11 || !alphas || !colors || !packed)
        return IGS_ERR_NULL_POINTER;
    if (!shape_ok(B, N, 1, 1)) return IGS_ERR_BAD_SHAPE;
    if (!channels_compiled(C)) return IGS_ERR_BAD_CHANNELS;
    const int Np = (N + 3) & ~3;
    hipLaunchKernelGGL((k_pack<false>), dim3(ceil_div(Np, kThreads), B), dim3(kThreads), 0,
                       (hipStream_t)stream, position, cov_inv_00, cov_inv_01, cov_inv_11, alphas,
                       colors, N, Np, C, rec_stride_of(C), 0.0f, packed,
                       const_cast<float4*>(boxes_of(packed, B, Np, rec_stride_of(C))), culling_enabled());
    return launch_status();
}

int igs_gs2d_pack_scale_rot(const float* positions, const float* scales, const float* rotations,
                            const float* alphas, const float* colors, int B, int N, int C, float eps,
                            float* packed, igs_stream_t stream) {
    if (!positions || !scales || !rotations || !alphas || !colors || !packed)
        return IGS_ERR_NULL_POINTER;
    if (!shape_ok(B, N, 1, 1)) return IGS_ERR_BAD_SHAPE;
    if (!channels_compiled(C)) return IGS_ERR_BAD_CHANNELS;
    const int Np = (N + 3) & ~3;
    hipLaunchKernelGGL((k_pack<true>), dim3(ceil_div(Np, kThreads), B), dim3(kThreads), 0,
                       (hipStream_t)stream, positions, scales, rotations, (const float*)nullptr,
                       alphas, colors, N, Np, C, rec_stride_of(C), eps, packed,
                       const_cast<float4*>(boxes_of(packed, B, Np, rec_stride_of(C))), culling_enabled());
    return launch_status();
}

int igs_gs2d_forward(const float* packed, const float* x, const float* y,
                     const int64_t grid_strides[6], int grid_mode, const int32_t* grid_flag, int B,
                     int N, int H, int W, int C, float eps, float* out, float* den, void* ws,
                     size_t ws_bytes, igs_stream_t stream) {
    if (!packed || !x || !y || !grid_strides || !out || !den) return IGS_ERR_NULL_POINTER;
    int rc = mode_ok(grid_mode, grid_flag);
    if (rc) return rc;
    if (!channels_compiled(C)) return IGS_ERR_BAD_CHANNELS;
    igs_gs2d_plan_t total;
    rc = make_plan(B, N, H, W, C, grid_mode, &total);
    if (rc) return rc;
    if (total.fwd_ws_bytes > 0 && (!ws || ws_bytes < total.fwd_ws_bytes)) return IGS_ERR_WORKSPACE;
    if (((uintptr_t)packed | (uintptr_t)ws) & 15) return IGS_ERR_ALIGNMENT;  // float4 / int lists inside
    hipStream_t st = (hipStream_t)stream;
    Variant vs[2];
    const int nv = variants_of(grid_mode, grid_flag, vs);
    for (int i = 0; i < nv; ++i) {
        igs_gs2d_plan_t plan;
        rc = plan_one(B, N, H, W, C, vs[i].mode, &plan);
        if (rc) return rc;
        const bool sep = vs[i].mode == IGS_GRID_SEPARABLE;
        const FwdGeometry fg = fwd_geometry(B, H, W, C, sep);
        FwdArgs a;
        a.packed = packed; a.x = x; a.y = y;
        a.sxb = grid_strides[0]; a.sxh = grid_strides[1]; a.sxw = grid_strides[2];
        a.syb = grid_strides[3]; a.syh = grid_strides[4]; a.syw = grid_strides[5];
        a.B = B; a.Np = plan.n_padded; a.H = H; a.W = W;
        a.S = plan.fwd_split;
        a.n_per_split = plan.fwd_n_per_split;
        a.tiles_x = fg.tiles_x; a.tiles_y = fg.tiles_y; a.total_tiles = fg.total_tiles; a.wx = fg.wx;
        a.eps = eps; a.out = out; a.den = den; a.part = (float*)ws;
        a.counts = nullptr; a.lists = nullptr;
        a.flag = vs[i].flag; a.want = vs[i].want;
        if (sep) {
            const size_t split_bytes = a.S > 1 ? (size_t)a.S * B * (C + 1) * H * W * sizeof(float) : 0;
            const BinPlace bp = bins_at(ws, split_bytes, B, plan.fwd_tiles);
            BinArgs ba;
            ba.boxes = boxes_of(packed, B, plan.n_padded, plan.rec_stride);
            ba.x = x; ba.y = y;
            ba.sxb = a.sxb; ba.sxw = a.sxw; ba.syb = a.syb; ba.syh = a.syh;
            ba.N = N; ba.Np = plan.n_padded; ba.H = H; ba.W = W;
            ba.tile_w = 64 * fg.wx; ba.tile_h = fwd_sep_p(C) * (4 / fg.wx);
            ba.tiles_x = fg.tiles_x; ba.tiles_y = fg.tiles_y;
            ba.counts = bp.counts; ba.lists = bp.lists; ba.slots = nullptr;
            ba.flag = vs[i].flag; ba.want = vs[i].want;
            rc = launch_bin(ba, B, st);
            if (rc) return rc;
            a.counts = bp.counts; a.lists = bp.lists;
        }
        IGS_DISPATCH_C(C, rc = launch_forward<kC>(a, sep, st));
        if (rc) return rc;
        if (a.S > 1) {
            hipLaunchKernelGGL(k_fwd_combine, dim3(ceil_div((long)H * W, kThreads), B), dim3(kThreads),
                               0, st, (const float*)ws, a.S, B, C, H * W, eps, out, den, a.flag, a.want);
            rc = launch_status();
            if (rc) return rc;
        }
    }
    return IGS_OK;
}

}  // extern "C"

namespace {
int backward_prologue(const float* x, const float* y, const int64_t grid_strides[6], int grid_mode,
                      const int32_t* grid_flag, const float* out, const float* den,
                      const float* grad_out, const MseArgs& mse, int B, int N, int H, int W, int C,
                      float eps, float* pix_ws, size_t pix_bytes, igs_stream_t stream) {
    if (!x || !y || !grid_strides || !out || !den || !pix_ws) return IGS_ERR_NULL_POINTER;
    if (!grad_out && !mse.target) return IGS_ERR_NULL_POINTER;
    int rc = mode_ok(grid_mode, grid_flag);
    if (rc) return rc;
    if (!channels_compiled(C)) return IGS_ERR_BAD_CHANNELS;
    igs_gs2d_plan_t total;
    rc = make_plan(B, N, H, W, C, grid_mode, &total);
    if (rc) return rc;
    if (pix_bytes < total.pix_bytes) return IGS_ERR_WORKSPACE;
    hipStream_t st = (hipStream_t)stream;
    Variant vs[2];
    const int nv = variants_of(grid_mode, grid_flag, vs);
    for (int i = 0; i < nv; ++i) {
        BwdArgs a;
        rc = bwd_args(a, vs[i], nullptr, nullptr, y, grid_strides, B, N, H, W, C, pix_ws, nullptr);
        if (rc) return rc;
        const bool sep = vs[i].mode == IGS_GRID_SEPARABLE;
        IGS_DISPATCH_C(C, rc = launch_bwd_prologue<kC>(a, B, sep, out, den, grad_out, mse, x, y, grid_strides, eps, pix_ws, st));
        if (rc) return rc;
    }
    return IGS_OK;
}
}  // namespace

extern "C" {

int igs_gs2d_backward_prologue(const float* x, const float* y, const int64_t grid_strides[6],
                               int grid_mode, const int32_t* grid_flag, const float* out,
                               const float* den, const float* grad_out, int B, int N, int H, int W,
                               int C, float eps, float* pix_ws, size_t pix_bytes,
                               igs_stream_t stream) {
    if (!grad_out) return IGS_ERR_NULL_POINTER;
    return backward_prologue(x, y, grid_strides, grid_mode, grid_flag, out, den, grad_out, MseArgs{}, B, N,
                             H, W, C, eps, pix_ws, pix_bytes, stream);
}

size_t igs_gs2d_mse_workspace_bytes(int B, int H, int W) {
    // one float per prologue workgroup of either grid variant (padded pixel counts differ)
    if (B < 1 || H < 1 || W < 1) return 0;
    const long sep = (long)H * ((W + 7) & ~7), gen = ((long)H * W + 3) & ~3L;
    return (size_t)B * ceil_div(sep > gen ? sep : gen, kThreads) * sizeof(float);
}

int igs_gs2d_backward_prologue_mse(const float* x, const float* y, const int64_t grid_strides[6],
                                   int grid_mode, const int32_t* grid_flag, const float* out,
                                   const float* den, const float* target, int C_real, int B, int N,
                                   int H, int W, int C, float eps, float* pix_ws, size_t pix_bytes,
                                   float* loss_ws, size_t loss_ws_bytes, float* loss,
                                   igs_stream_t stream) {
    if (!target || !loss_ws || !loss) return IGS_ERR_NULL_POINTER;
    if (C_real < 1 || C_real > C) return IGS_ERR_BAD_SHAPE;
    if (loss_ws_bytes < igs_gs2d_mse_workspace_bytes(B, H, W)) return IGS_ERR_WORKSPACE;
    MseArgs mse;
    const double count = (double)B * C_real * H * W;
    mse.target = target;
    mse.gscale = (float)(2.0 / count);
    mse.loss_part = loss_ws;
    mse.loss_scale = (float)(1.0 / count);
    mse.loss = loss;
    return backward_prologue(x, y, grid_strides, grid_mode, grid_flag, out, den, nullptr, mse, B, N, H, W,
                             C, eps, pix_ws, pix_bytes, stream);
}

int igs_adamw_step(float* param, const float* grad, float* exp_avg, float* exp_avg_sq, int64_t count,
                   float* state, float beta1, float beta2, float eps, float weight_decay,
                   igs_stream_t stream) {
    if (!param || !grad || !exp_avg || !exp_avg_sq || !state) return IGS_ERR_NULL_POINTER;
    if (count < 1 || count > (int64_t)kThreads * 0x7fffffff) return IGS_ERR_BAD_SHAPE;
    hipStream_t st = (hipStream_t)stream;
    hipLaunchKernelGGL(k_adamw_tick, dim3(1), dim3(64), 0, st, state, beta1, beta2);
    int rc = launch_status();
    if (rc) return rc;
    hipLaunchKernelGGL(k_adamw, dim3((unsigned)((count + kThreads - 1) / kThreads)), dim3(kThreads), 0, st,
                       param, grad, exp_avg, exp_avg_sq, (long)count, state, beta1, beta2, eps, weight_decay);
    return launch_status();
}

int igs_gs2d_backward_reduce(const float* packed, const float* colors, const float* y,
                             const int64_t grid_strides[6], int grid_mode, const int32_t* grid_flag,
                             int B, int N, int H, int W, int C, float* pix_ws, size_t pix_bytes,
                             float* partial, size_t partial_bytes, igs_stream_t stream) {
    if (!packed || !colors || !y || !grid_strides || !pix_ws || !partial) return IGS_ERR_NULL_POINTER;
    int rc = mode_ok(grid_mode, grid_flag);
    if (rc) return rc;
    if (!channels_compiled(C)) return IGS_ERR_BAD_CHANNELS;
    igs_gs2d_plan_t total;
    rc = make_plan(B, N, H, W, C, grid_mode, &total);
    if (rc) return rc;
    if (pix_bytes < total.pix_bytes || partial_bytes < total.partial_bytes) return IGS_ERR_WORKSPACE;
    if (((uintptr_t)packed | (uintptr_t)pix_ws) & 15) return IGS_ERR_ALIGNMENT;  // float4 / int lists inside
    hipStream_t st = (hipStream_t)stream;
    Variant vs[2];
    const int nv = variants_of(grid_mode, grid_flag, vs);
    for (int i = 0; i < nv; ++i) {
        BwdArgs a;
        rc = bwd_args(a, vs[i], packed, colors, y, grid_strides, B, N, H, W, C, pix_ws, partial);
        if (rc) return rc;
        const bool sep = vs[i].mode == IGS_GRID_SEPARABLE;
        if (sep) {
            BinArgs ba;
            ba.boxes = boxes_of(packed, B, a.Np, rec_stride_of(C));
            ba.x = a.xs; ba.y = y;               // the prologue's compact column coordinates
            ba.sxb = a.Wp; ba.sxw = 1; ba.syb = a.syb; ba.syh = a.syh;
            ba.N = N; ba.Np = a.Np; ba.H = H; ba.W = W;
            ba.tile_w = kBwdTileW; ba.tile_h = a.per_tile;
            ba.tiles_x = a.tiles_x; ba.tiles_y = a.T / a.tiles_x;
            ba.counts = const_cast<int*>(a.counts); ba.lists = const_cast<int*>(a.lists);
            ba.slots = slots_at(partial, B, a.T, 6 + C, N);
            ba.flag = a.flag; ba.want = a.want;
            rc = launch_bin(ba, B, st);
            if (rc) return rc;
        }
        IGS_DISPATCH_C(C, rc = launch_bwd_reduce<kC>(a, B, sep, st));
        if (rc) return rc;
    }
    return IGS_OK;
}

int igs_gs2d_backward(const float* packed, const float* colors, const float* x, const float* y,
                      const int64_t grid_strides[6], int grid_mode, const int32_t* grid_flag,
                      const float* out, const float* den, const float* grad_out, int B, int N, int H,
                      int W, int C, float eps, float* pix_ws, size_t pix_bytes, float* partial,
                      size_t partial_bytes, igs_stream_t stream) {
    int rc = igs_gs2d_backward_prologue(x, y, grid_strides, grid_mode, grid_flag, out, den, grad_out, B, N,
                                        H, W, C, eps, pix_ws, pix_bytes, stream);
    if (rc) return rc;
    return igs_gs2d_backward_reduce(packed, colors, y, grid_strides, grid_mode, grid_flag, B, N, H, W, C,
                                    pix_ws, pix_bytes, partial, partial_bytes, stream);
}

int igs_gs2d_backward_grid(const float* packed, const float* x, const float* y,
                           const int64_t grid_strides[6], const float* out, const float* den,
                           const float* grad_out, int B, int N, int H, int W, int C, float eps,
                           float* g_x, float* g_y, igs_stream_t stream) {
    if (!packed || !x || !y || !grid_strides || !out || !den || !grad_out || !g_x || !g_y)
        return IGS_ERR_NULL_POINTER;
    if (!shape_ok(B, N, H, W)) return IGS_ERR_BAD_SHAPE;
    if (!channels_compiled(C)) return IGS_ERR_BAD_CHANNELS;
    GridGradArgs a;
    a.packed = packed; a.x = x; a.y = y;
    a.sxb = grid_strides[0]; a.sxh = grid_strides[1]; a.sxw = grid_strides[2];
    a.syb = grid_strides[3]; a.syh = grid_strides[4]; a.syw = grid_strides[5];
    a.out = out; a.den = den; a.gout = grad_out;
    a.Np = (N + 3) & ~3; a.H = H; a.W = W;
    a.eps = eps; a.gx = g_x; a.gy = g_y;
    int rc = IGS_OK;
    hipStream_t st = (hipStream_t)stream;
    IGS_DISPATCH_C(C, {
        constexpr int P = kC > 8 ? 2 : 4;
        a.tiles_per_img = ceil_div((long)H * W, kThreads * P);
        a.total_tiles = B * a.tiles_per_img;
        hipLaunchKernelGGL((k_bwd_grid<kC, P>), dim3(((a.total_tiles + 7) / 8) * 8), dim3(kThreads), 0, st, a);
        rc = launch_status();
    });
    return rc;
}

// The slot tables that the separable backward left behind the partial sums (none on general grids).
static const int* finalize_slots(const float* partial, int grid_mode, int B, int T, int NF, int N) {
    if (grid_mode == IGS_GRID_GENERAL) return nullptr;
    return slots_at(const_cast<float*>(partial), B, T, NF, N);
}

// T of the separable (or only) variant and of the general variant under AUTO.
static int finalize_tiles(int grid_mode, int B, int N, int H, int W, int C, int* T, int* T_alt) {
    igs_gs2d_plan_t plan;
    int rc = plan_one(B, N, H, W, C, grid_mode == IGS_GRID_AUTO ? IGS_GRID_SEPARABLE : grid_mode, &plan);
    if (rc) return rc;
    *T = plan.bwd_tiles;
    *T_alt = plan.bwd_tiles;
    if (grid_mode == IGS_GRID_AUTO) {
        rc = plan_one(B, N, H, W, C, IGS_GRID_GENERAL, &plan);
        if (rc) return rc;
        *T_alt = plan.bwd_tiles;
    }
    return IGS_OK;
}

int igs_gs2d_finalize_covinv(const float* partial, int grid_mode, const int32_t* grid_flag,
                             const float* cov_inv_00, const float* cov_inv_01,
                             const float* cov_inv_11, const float* alphas, int B, int N, int H, int W,
                             int C, float* g_position, float* g_cov_inv_00, float* g_cov_inv_01,
                             float* g_cov_inv_11, float* g_alphas, float* g_colors,
                             igs_stream_t stream) {
    if (!partial || !cov_inv_00 || !cov_inv_01 || !cov_inv_11 || !alphas) return IGS_ERR_NULL_POINTER;
    int rc = mode_ok(grid_mode, grid_flag);
    if (rc) return rc;
    int T, T_alt;
    rc = finalize_tiles(grid_mode, B, N, H, W, C, &T, &T_alt);
    if (rc) return rc;
    hipLaunchKernelGGL((k_bwd_finalize<false>), dim3(ceil_div(N, kFinN), B), dim3(kThreads), 0,
                       (hipStream_t)stream, partial, T, grid_mode == IGS_GRID_AUTO ? grid_flag : nullptr,
                       T_alt, finalize_slots(partial, grid_mode, B, T, 6 + C, N), (N + 3) & ~3, cov_inv_00,
                       cov_inv_01, cov_inv_11, alphas, N, C, 0.0f, g_position,
                       g_cov_inv_00, g_cov_inv_01, g_cov_inv_11, g_alphas, g_colors);
    return launch_status();
}

int igs_gs2d_finalize_scale_rot(const float* partial, int grid_mode, const int32_t* grid_flag,
                                const float* scales, const float* rotations, const float* alphas,
                                int B, int N, int H, int W, int C, float eps, float* g_positions,
                                float* g_scales, float* g_rotations, float* g_alphas, float* g_colors,
                                igs_stream_t stream) {
    if (!partial || !scales || !rotations || !alphas) return IGS_ERR_NULL_POINTER;
    int rc = mode_ok(grid_mode, grid_flag);
    if (rc) return rc;
    int T, T_alt;
    rc = finalize_tiles(grid_mode, B, N, H, W, C, &T, &T_alt);
    if (rc) return rc;
    hipLaunchKernelGGL((k_bwd_finalize<true>), dim3(ceil_div(N, kFinN), B), dim3(kThreads), 0,
                       (hipStream_t)stream, partial, T, grid_mode == IGS_GRID_AUTO ? grid_flag : nullptr,
                       T_alt, finalize_slots(partial, grid_mode, B, T, 6 + C, N), (N + 3) & ~3, scales, rotations,
                       (const float*)nullptr, alphas, N, C, eps, g_positions,
                       g_scales, g_rotations, (float*)nullptr, g_alphas, g_colors);
    return launch_status();
}

int igs_gs2d_pack_feature(const float* gs_feature, const float* pos_offset, int B, int N, int C,
                          int C_kernel, float eps, float* packed, float* colors_out,
                          igs_stream_t stream) {
    if (!gs_feature || !packed || !colors_out) return IGS_ERR_NULL_POINTER;
    if (!shape_ok(B, N, 1, 1)) return IGS_ERR_BAD_SHAPE;
    if (C < 1 || C > C_kernel || !channels_compiled(C_kernel)) return IGS_ERR_BAD_CHANNELS;
    const int Np = (N + 3) & ~3;
    hipLaunchKernelGGL(k_pack_feature, dim3(ceil_div(Np, kThreads), B), dim3(kThreads), 0,
                       (hipStream_t)stream, gs_feature, pos_offset, N, Np, C, C_kernel,
                       rec_stride_of(C_kernel), eps, packed,
                       const_cast<float4*>(boxes_of(packed, B, Np, rec_stride_of(C_kernel))), colors_out,
                       culling_enabled());
    return launch_status();
}

int igs_gs2d_finalize_feature(const float* partial, int grid_mode, const int32_t* grid_flag,
                              const float* gs_feature, int B, int N, int H, int W, int C,
                              int C_kernel, float eps, float* g_feature, igs_stream_t stream) {
    if (!partial || !gs_feature || !g_feature) return IGS_ERR_NULL_POINTER;
    int rc = mode_ok(grid_mode, grid_flag);
    if (rc) return rc;
    if (C < 1 || C > C_kernel || !channels_compiled(C_kernel)) return IGS_ERR_BAD_CHANNELS;
    int T, T_alt;
    rc = finalize_tiles(grid_mode, B, N, H, W, C_kernel, &T, &T_alt);
    if (rc) return rc;
    hipLaunchKernelGGL(k_bwd_finalize_feature, dim3(ceil_div(N, kFinN), B), dim3(kThreads), 0,
                       (hipStream_t)stream, partial, T, grid_mode == IGS_GRID_AUTO ? grid_flag : nullptr,
                       T_alt, finalize_slots(partial, grid_mode, B, T, 6 + C_kernel, N), (N + 3) & ~3, gs_feature,
                       N, C, C_kernel, eps, g_feature);
    return launch_status();
}

}  // extern "C"
