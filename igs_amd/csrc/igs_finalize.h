// igs_finalize.h -- finalize kernels: fixed-order sum of the tile partials and the chain rule.
// Included by igs_gs2d.hip inside its anonymous namespace (one translation unit).
#pragma once

// Fixed-order sum over the T tile partials of NV consecutive fields for one Gaussian, spread
// over the FT "t-lanes" of a workgroup laid out as FT t-lanes x FN = 256/FT Gaussians: t-lane k
// adds tiles k, k+FT, ... in order, the lane sums are then added in order by every thread (so
// all t-lanes of a Gaussian hold the same, run-to-run identical value).  `red` is
// [NV][FT][FN+1] floats of LDS.  Must be called by all 256 threads.  Two layouts are compiled:
// 8 x 32 (the consecutive Gaussians of a wave read neighbouring columns of a tile's partials)
// and, for problems too small to fill the device with that one, 32 x 8 (the sequential,
// latency-bound part of a sum over hundreds of tiles gets 4 times shorter; timed against 16 and 64).
#ifndef IGS_FIN_DEEP
#define IGS_FIN_DEEP 32
#endif
constexpr int kFinWide = 8, kFinDeep = IGS_FIN_DEEP;
constexpr int kFinAhead = 4;    // tiles whose loads are issued together by a t-lane
constexpr int kFinColours = 8;  // colour channels summed per further pass
constexpr int kFinFirst = 9;    // fields of the first pass: the six moments and up to three colours (C <= 3: one pass)

// `part` is the image's partial array [T][N][NF]; the Gaussian's column in tile t is
// slots[t * Np + n] when a slot table is given (negative: the tile holds nothing for it), else n.
// Only the first `nv` (<= NV) of the fields are read.
template <int NV, int FT>
__device__ __forceinline__ void tile_sum(const float* __restrict__ part, const int* __restrict__ slots,
                                         int Np, int n, int T, int NF, int N, int f0, bool valid,
                                         float (&out)[NV], float* red, int nv = NV) {
    constexpr int FN = 256 / FT;
    const int tl = threadIdx.x / FN, nl = threadIdx.x % FN;
    float acc[NV];
#pragma unroll
    for (int v = 0; v < NV; ++v) acc[v] = 0.0f;
    if (valid) {
        // kFinAhead tiles at a time: their slot entries first, then all their partials (loads of
        // absent entries go to column 0 and are replaced by 0), then the sums in tile order, so that
        // the loads of a group are in flight together instead of one dependent pair after the other
        for (int t0 = tl; t0 < T; t0 += FT * kFinAhead) {
            int col[kFinAhead];
#pragma unroll
            for (int u = 0; u < kFinAhead; ++u) {
                const int t = t0 + u * FT;
                col[u] = t < T ? (slots ? slots[(size_t)t * Np + n] : n) : -1;
            }
            float val[kFinAhead][NV];
#pragma unroll
            for (int u = 0; u < kFinAhead; ++u) {
                const int t = min(t0 + u * FT, T - 1);
                const float* src = part + ((size_t)t * N + max(col[u], 0)) * NF + f0;
#pragma unroll
                for (int v = 0; v < NV; ++v) val[u][v] = v < nv ? src[v] : 0.0f;
            }
#pragma unroll
            for (int u = 0; u < kFinAhead; ++u)
#pragma unroll
                for (int v = 0; v < NV; ++v) acc[v] += col[u] >= 0 ? val[u][v] : 0.0f;
        }
    }
    __syncthreads();  // protects `red` against the previous call's readers
#pragma unroll
    for (int v = 0; v < NV; ++v) red[(v * FT + tl) * (FN + 1) + nl] = acc[v];
    __syncthreads();
#pragma unroll
    for (int v = 0; v < NV; ++v) {
        float s = 0.0f;
#pragma unroll
        for (int k = 0; k < FT; ++k) s += red[(v * FT + k) * (FN + 1) + nl];
        out[v] = s;
    }
}

// The same sum after a two-level binning: a tile's slot entry exists only where the super-tile
// lists the Gaussian (cslots[st][n] >= 0), so the t-lanes walk the super-tiles (t-lane k takes
// k, k + FT, ...) and, in a listed one, its tiles row by row (the four tiles of a row together).
// A Gaussian reaches a few super-tiles, so this reads a fraction of the slot tables.
struct SuperSlots {
    const int* cslots;  // this image's [stiles][Np]; nullptr: one-level binning
    int tiles_x, tiles_y, stiles_x, stiles;
};

template <int NV, int FT>
__device__ __forceinline__ void tile_sum_super(const float* __restrict__ part, const int* __restrict__ slots,
                                               const SuperSlots sup, int Np, int n, int NF, int N, int f0,
                                               bool valid, float (&out)[NV], float* red, int nv = NV) {
    constexpr int FN = 256 / FT;
    const int tl = threadIdx.x / FN, nl = threadIdx.x % FN;
    float acc[NV];
#pragma unroll
    for (int v = 0; v < NV; ++v) acc[v] = 0.0f;
    if (valid) {
        for (int st = tl; st < sup.stiles; st += FT) {
            if (sup.cslots[(size_t)st * Np + n] < 0) continue;
            const int sy = st / sup.stiles_x, sx = st - sy * sup.stiles_x;
            for (int j = 0; j < kSuperY; ++j) {
                const int ty = sy * kSuperY + j;
                if (ty >= sup.tiles_y) break;
                int col[kSuperX];
#pragma unroll
                for (int u = 0; u < kSuperX; ++u) {
                    const int tx = sx * kSuperX + u;
                    col[u] = tx < sup.tiles_x ? slots[(size_t)(ty * sup.tiles_x + tx) * Np + n] : -1;
                }
                float val[kSuperX][NV];
#pragma unroll
                for (int u = 0; u < kSuperX; ++u) {
                    const int t = ty * sup.tiles_x + min(sx * kSuperX + u, sup.tiles_x - 1);
                    const float* src = part + ((size_t)t * N + max(col[u], 0)) * NF + f0;
#pragma unroll
                    for (int v = 0; v < NV; ++v) val[u][v] = v < nv ? src[v] : 0.0f;
                }
#pragma unroll
                for (int u = 0; u < kSuperX; ++u)
#pragma unroll
                    for (int v = 0; v < NV; ++v) acc[v] += col[u] >= 0 ? val[u][v] : 0.0f;
            }
        }
    }
    __syncthreads();  // protects `red` against the previous call's readers
#pragma unroll
    for (int v = 0; v < NV; ++v) red[(v * FT + tl) * (FN + 1) + nl] = acc[v];
    __syncthreads();
#pragma unroll
    for (int v = 0; v < NV; ++v) {
        float s = 0.0f;
#pragma unroll
        for (int k = 0; k < FT; ++k) s += red[(v * FT + k) * (FN + 1) + nl];
        out[v] = s;
    }
}

// Finalize: FT threads per Gaussian; sums the T tile partials in a fixed order and applies
//   d alpha = M0, d color_c = alpha CG_c, d px = alpha (A Mx + B My), d py = alpha (B Mx + D My),
//   dA = -1/2 alpha Mxx, dB = -alpha Mxy, dD = -1/2 alpha Myy,
// and (function level) the chain rule through A = c^2 i0 + s^2 i1, B = c s (i0 - i1),
// D = s^2 i0 + c^2 i1, i_k = 1/(s_k^2 + eps).
template <bool kScaleRot, int FT>
__global__ __launch_bounds__(kThreads) void k_bwd_finalize(
    const float* __restrict__ partial, int T_in, const int* __restrict__ flag, int T_alt,
    const int* __restrict__ slots_in, const SuperSlots sup_in, int Np, const float* __restrict__ p0,
    const float* __restrict__ p1, const float* __restrict__ p2, const float* __restrict__ alphas,
    int N, int C, float eps, float* __restrict__ g_pos, float* __restrict__ g0,
    float* __restrict__ g1, float* __restrict__ g2, float* __restrict__ g_alpha,
    float* __restrict__ g_col) {
    constexpr int FN = 256 / FT;
    __shared__ float red[kFinFirst * FT * (FN + 1)];
    const int n = blockIdx.x * FN + threadIdx.x % FN;
    const int b = blockIdx.y;
    const bool valid = n < N;
    const bool writer = valid && threadIdx.x < FN;  // t-lane 0 writes the results
    // AUTO grid mode: T_in belongs to the separable plan, T_alt to the general one
    const int T = (flag != nullptr && *flag == 0) ? T_alt : T_in;
    const int NF = 6 + C;
    const size_t i = (size_t)b * N + min(n, N - 1);
    const float* part = partial + (size_t)b * T * NF * N;
    // the slot table belongs to the separable variant
    const int* slots = (slots_in != nullptr && !(flag != nullptr && *flag == 0))
                           ? slots_in + (size_t)b * T * Np : nullptr;
    SuperSlots sup = sup_in;  // the super-tile tables belong to the separable variant as well
    sup.cslots = (slots != nullptr && sup_in.cslots != nullptr) ? sup_in.cslots + (size_t)b * sup_in.stiles * Np : nullptr;
    const int nn = min(n, N - 1);
    // first pass: the moments and, when wanted, the first colours (they follow the moments)
    constexpr int kC0 = kFinFirst - 6;
    float M[kFinFirst];
    const int nfirst = g_col ? min(kFinFirst, NF) : 6;
    if (sup.cslots != nullptr)  // kernel-argument and flag uniform: the barriers inside are safe
        tile_sum_super<kFinFirst, FT>(part, slots, sup, Np, nn, NF, N, 0, valid, M, red, nfirst);
    else
        tile_sum<kFinFirst, FT>(part, slots, Np, nn, T, NF, N, 0, valid, M, red, nfirst);
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
        if (writer)
#pragma unroll
            for (int c = 0; c < kC0; ++c)
                if (c < C) g_col[i * C + c] = (float)al * M[6 + c];
        for (int c0 = kC0; c0 < C; c0 += kFinColours) {  // further colour sums, kFinColours channels per pass
            float sc[kFinColours];
            const int nc = min(kFinColours, C - c0);
            if (sup.cslots != nullptr)
                tile_sum_super<kFinColours, FT>(part, slots, sup, Np, nn, NF, N, 6 + c0, valid, sc, red, nc);
            else
                tile_sum<kFinColours, FT>(part, slots, Np, nn, T, NF, N, 6 + c0, valid, sc, red, nc);
            if (writer)
#pragma unroll
                for (int c = 0; c < kFinColours; ++c)
                    if (c < nc) g_col[i * C + c0 + c] = (float)al * sc[c];
        }
    }
}

// Finalize for the fused module head: d gs_feature [B][N][6+C] from the tile partials, with
// alpha = 1, d log_s_k = d s_k * exp(log_s_k) and a zero gradient for the unused opacity logit.
template <int FT>
__global__ __launch_bounds__(kThreads) void k_bwd_finalize_feature(
    const float* __restrict__ partial, int T_in, const int* __restrict__ flag, int T_alt,
    const int* __restrict__ slots_in, const SuperSlots sup_in, int Np, const float* __restrict__ feat, int N,
    int C, int Cp,
    float eps, float* __restrict__ g_feat) {
    constexpr int FN = 256 / FT;
    __shared__ float red[kFinFirst * FT * (FN + 1)];
    const int n = blockIdx.x * FN + threadIdx.x % FN;
    const int b = blockIdx.y;
    const bool valid = n < N;
    const bool writer = valid && threadIdx.x < FN;
    const int T = (flag != nullptr && *flag == 0) ? T_alt : T_in;
    const int NF = 6 + Cp;
    const size_t i = (size_t)b * N + min(n, N - 1);
    const float* part = partial + (size_t)b * T * NF * N;
    const int* slots = (slots_in != nullptr && !(flag != nullptr && *flag == 0))
                           ? slots_in + (size_t)b * T * Np : nullptr;
    SuperSlots sup = sup_in;  // the super-tile tables belong to the separable variant as well
    sup.cslots = (slots != nullptr && sup_in.cslots != nullptr) ? sup_in.cslots + (size_t)b * sup_in.stiles * Np : nullptr;
    const int nn = min(n, N - 1);
    constexpr int kC0 = kFinFirst - 6;
    float M[kFinFirst];
    if (sup.cslots != nullptr)  // kernel-argument and flag uniform: the barriers inside are safe
        tile_sum_super<kFinFirst, FT>(part, slots, sup, Np, nn, NF, N, 0, valid, M, red, min(kFinFirst, NF));
    else
        tile_sum<kFinFirst, FT>(part, slots, Np, nn, T, NF, N, 0, valid, M, red, min(kFinFirst, NF));
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
#pragma unroll
        for (int c = 0; c < kC0; ++c)
            if (c < C) g[6 + c] = M[6 + c];
    }
    for (int c0 = kC0; c0 < C; c0 += kFinColours) {
        float sc[kFinColours];
        const int nc = min(kFinColours, C - c0);
        if (sup.cslots != nullptr)
            tile_sum_super<kFinColours, FT>(part, slots, sup, Np, nn, NF, N, 6 + c0, valid, sc, red, nc);
        else
            tile_sum<kFinColours, FT>(part, slots, Np, nn, T, NF, N, 6 + c0, valid, sc, red, nc);
        if (writer)
#pragma unroll
            for (int c = 0; c < kFinColours; ++c)
                if (c < nc) g[6 + c0 + c] = sc[c];
    }
}
