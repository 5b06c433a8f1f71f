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

// General grids: `part` is the image's partial array [T][N][NF] and the Gaussian's column in every tile
// is n (slots, toff: nullptr).  Separable grids: `part` is the compact array of all images, tile t of
// this image starts at record toff[t], and the Gaussian's record in it is number slots[t * Np + n]
// (negative: the tile holds nothing for it).  Only the first `nv` (<= NV) of the fields are read.
template <int NV, int FT>
__device__ __forceinline__ void tile_sum(const float* __restrict__ part, const int* __restrict__ slots,
                                         const long long* __restrict__ toff,
                                         int Np, int n, int T, int NF, int N, int f0, bool valid,
                                         float (&out)[NV], float* red, int nv = NV) {
    constexpr int FN = 256 / FT;
    const int tl = threadIdx.x / FN, nl = threadIdx.x % FN;
    float acc[NV];
#pragma unroll
    for (int v = 0; v < NV; ++v) acc[v] = 0.0f;
    if (valid) {
        // kFinAhead tiles at a time: their slot entries first, then all their partials (loads of
        // absent entries go to the array's first record and are replaced by 0), then the sums in tile order, so that
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
                const size_t record = slots ? (col[u] >= 0 ? (size_t)(toff[t] + col[u]) : (size_t)0)
                                            : (size_t)t * N + max(col[u], 0);
                const float* src = part + record * NF + f0;
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

// The tables of a two-level binning: a tile's slot entry exists only where the super-tile lists
// the Gaussian (cslots[st][n] >= 0).
struct SuperSlots {
    const int* cslots;  // [B][stiles][Np]; nullptr: one-level binning
    int tiles_x, tiles_y, stiles_x, stiles;
};

// Chain rule of the operator and function level for one Gaussian (i = b N + n), from its six
// moment sums M = (M0, Mx, My, Mxx, Mxy, Myy):
//   d alpha = M0, d px = alpha (A Mx + B My), d py = alpha (B Mx + D My),
//   dA = -1/2 alpha Mxx, dB = -alpha Mxy, dD = -1/2 alpha Myy,
// and (function level) through A = c^2 i0 + s^2 i1, B = c s (i0 - i1), D = s^2 i0 + c^2 i1,
// i_k = 1/(s_k^2 + eps).  In fp64: the chain rule multiplies sums by 1/s^3-sized factors.
template <bool kScaleRot>
__device__ __forceinline__ void finalize_geometry(const float* M, size_t i, const float* __restrict__ p0,
                                                  const float* __restrict__ p1, const float* __restrict__ p2,
                                                  const float* __restrict__ alphas, float eps,
                                                  float* __restrict__ g_pos, float* __restrict__ g0,
                                                  float* __restrict__ g1, float* __restrict__ g2,
                                                  float* __restrict__ g_alpha) {
    const double al = alphas[i];
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
    if (g_alpha) g_alpha[i] = M[0];
    if (g_pos) {
        g_pos[2 * i] = (float)(al * (A * M[1] + Bc * M[2]));
        g_pos[2 * i + 1] = (float)(al * (Bc * M[1] + D * M[2]));
    }
    const double gA = -0.5 * al * M[3], gB = -al * M[4], gD = -0.5 * al * M[5];
    if (kScaleRot) {
        if (g0) {  // scales [B,N,2]
            const double gi0 = gA * cs * cs + gB * cs * sn + gD * sn * sn;
            const double gi1 = gA * sn * sn - gB * cs * sn + gD * cs * cs;
            g0[2 * i] = (float)(gi0 * (-2.0 * s0 * i0 * i0));
            g0[2 * i + 1] = (float)(gi1 * (-2.0 * s1 * i1 * i1));
        }
        if (g1) g1[i] = (float)((gD - gA) * 2.0 * Bc + gB * (cs * cs - sn * sn) * (i0 - i1));
    } else {
        if (g0) g0[i] = (float)gA;
        if (g1) g1[i] = (float)gB;
        if (g2) g2[i] = (float)gD;
    }
}

// The same for the fused module head: d gs_feature[0..5] of one Gaussian (f, g: its rows of
// 6 + C floats), with alpha = 1, d log_s_k = d s_k * exp(log_s_k) and a zero gradient for the
// unused opacity logit.
__device__ __forceinline__ void finalize_feature_geometry(const float* M, const float* __restrict__ f, float eps,
                                                          float* __restrict__ g) {
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
    g[0] = (float)(A * M[1] + Bc * M[2]);
    g[1] = (float)(Bc * M[1] + D * M[2]);
    g[2] = (float)(gi0 * (-2.0 * s0 * i0 * i0) * e0);
    g[3] = (float)(gi1 * (-2.0 * s1 * i1 * i1) * e1);
    g[4] = (float)((gD - gA) * 2.0 * Bc + gB * (cs * cs - sn * sn) * (i0 - i1));
    g[5] = 0.0f;
}

// Finalize: FT threads per Gaussian; sums the T tile partials in a fixed order and applies the
// chain rule (finalize_geometry; d color_c = alpha CG_c).  For one-level tile lists and for
// general grids; after a two-level binning k_bwd_finalize_listed runs instead.
template <bool kScaleRot, int FT>
__global__ __launch_bounds__(kThreads) void k_bwd_finalize(
    const float* __restrict__ partial, int T_in, const int* __restrict__ flag, int T_alt,
    const int* __restrict__ slots_in, const long long* __restrict__ offsets, const int* __restrict__ overflow,
    int stamp, int Np, const float* __restrict__ p0,
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
    // the slot table and the compact array belong to the separable variant
    const bool listed = slots_in != nullptr && !(flag != nullptr && *flag == 0);
    const int* slots = listed ? slots_in + (size_t)b * T * Np : nullptr;
    const long long* toff = listed ? offsets + (size_t)b * T : nullptr;
    const float* part = listed ? partial : partial + (size_t)b * T * NF * N;
    // the partial sums did not fit the caller's array, or the tables are not this problem's: no gradient is known
    const bool lost = listed && (overflow[0] != 0 || overflow[1] != stamp);
    const int nn = min(n, N - 1);
    // first pass: the moments and, when wanted, the first colours (they follow the moments)
    constexpr int kC0 = kFinFirst - 6;
    float M[kFinFirst];
    const int nfirst = g_col ? min(kFinFirst, NF) : 6;
    tile_sum<kFinFirst, FT>(part, slots, toff, Np, nn, T, NF, N, 0, valid && !lost, M, red, nfirst);
    if (lost)
#pragma unroll
        for (int v = 0; v < kFinFirst; ++v) M[v] = __builtin_nanf("");
    if (writer) finalize_geometry<kScaleRot>(M, i, p0, p1, p2, alphas, eps, g_pos, g0, g1, g2, g_alpha);
    if (g_col) {  // kernel-argument uniform, so the barriers inside tile_sum are safe
        const float al = alphas[i];
        if (writer)
#pragma unroll
            for (int c = 0; c < kC0; ++c)
                if (c < C) g_col[i * C + c] = al * M[6 + c];
        for (int c0 = kC0; c0 < C; c0 += kFinColours) {  // further colour sums, kFinColours channels per pass
            float sc[kFinColours];
            const int nc = min(kFinColours, C - c0);
            tile_sum<kFinColours, FT>(part, slots, toff, Np, nn, T, NF, N, 6 + c0, valid && !lost, sc, red, nc);
            if (writer)
#pragma unroll
                for (int c = 0; c < kFinColours; ++c)
                    if (c < nc) g_col[i * C + c0 + c] = lost ? __builtin_nanf("") : al * sc[c];
        }
    }
}

// Finalize for the fused module head: d gs_feature [B][N][6+C] from the tile partials
// (finalize_feature_geometry; d colour_c = CG_c).
template <int FT>
__global__ __launch_bounds__(kThreads) void k_bwd_finalize_feature(
    const float* __restrict__ partial, int T_in, const int* __restrict__ flag, int T_alt,
    const int* __restrict__ slots_in, const long long* __restrict__ offsets, const int* __restrict__ overflow,
    int stamp, int Np, const float* __restrict__ feat, int N,
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
    const bool listed = slots_in != nullptr && !(flag != nullptr && *flag == 0);
    const int* slots = listed ? slots_in + (size_t)b * T * Np : nullptr;
    const long long* toff = listed ? offsets + (size_t)b * T : nullptr;
    const float* part = listed ? partial : partial + (size_t)b * T * NF * N;
    const bool lost = listed && (overflow[0] != 0 || overflow[1] != stamp);
    const int nn = min(n, N - 1);
    constexpr int kC0 = kFinFirst - 6;
    float M[kFinFirst];
    tile_sum<kFinFirst, FT>(part, slots, toff, Np, nn, T, NF, N, 0, valid && !lost, M, red, min(kFinFirst, NF));
    if (lost)
#pragma unroll
        for (int v = 0; v < kFinFirst; ++v) M[v] = __builtin_nanf("");
    float* g = g_feat + i * (6 + C);
    if (writer) {
        finalize_feature_geometry(M, feat + i * (6 + C), eps, g);
#pragma unroll
        for (int c = 0; c < kC0; ++c)
            if (c < C) g[6 + c] = M[6 + c];
    }
    for (int c0 = kC0; c0 < C; c0 += kFinColours) {
        float sc[kFinColours];
        const int nc = min(kFinColours, C - c0);
        tile_sum<kFinColours, FT>(part, slots, toff, Np, nn, T, NF, N, 6 + c0, valid && !lost, sc, red, nc);
        if (writer)
#pragma unroll
            for (int c = 0; c < kFinColours; ++c)
                if (c < nc) g[6 + c0 + c] = lost ? __builtin_nanf("") : sc[c];
    }
}

// ------------------------------------------------------------------ after a two-level binning
// Sparse scenes: a Gaussian is listed in a few of hundreds of tiles, and consecutive Gaussians in
// different ones, so a thread per Gaussian reads each record of 6 + C floats with 6 + C scattered
// loads while most lanes of its wave idle (c4, C = 16: 236 us).  Here a group of 8 lanes works on
// one Gaussian: its lanes test 8 super-tiles, then 8 tiles of a listed super-tile, with one load
// instruction each, and read a record as contiguous runs of 8 floats (lane v holds fields v, v + 8,
// v + 16).  A workgroup takes 32 Gaussians, one per group; the moments go through LDS to the chain
// rule, which 32 threads then evaluate for one Gaussian each, and the lanes that hold colour sums
// write the colour gradients themselves.  Tiles are added in ascending super-tile, then row-major
// tile order: a fixed order.  Timed at c4 (131072 Gaussians, 960 tiles): groups of 8 / 16 / 32 lanes
// 93 / 103 / 120 us, 32 against 64 Gaussians per workgroup 93 against 108.
#ifndef IGS_FIN_GROUP
#define IGS_FIN_GROUP 8
#endif
#ifndef IGS_FIN_GROUP_AHEAD
#define IGS_FIN_GROUP_AHEAD 4
#endif
#ifndef IGS_FIN_GROUP_BATCH
#define IGS_FIN_GROUP_BATCH 32
#endif
constexpr int kFinGroup = IGS_FIN_GROUP;             // lanes per Gaussian
constexpr int kFinGroupBatch = IGS_FIN_GROUP_BATCH;  // Gaussians per workgroup
constexpr int kFinGroupAhead = IGS_FIN_GROUP_AHEAD;  // records whose loads a group issues together
constexpr int kFinGroupFields = (6 + IGS_MAX_CHANNELS + kFinGroup - 1) / kFinGroup;  // fields per lane: lane, lane + kFinGroup, ..
static_assert(kFinGroup == 8 || kFinGroup == 16 || kFinGroup == 32, "a power of two that divides a half wave");

struct FinalizeArgs {
    const float* partial;
    int T, T_alt;
    const int* flag;    // AUTO grid mode: *flag == 0 -> the general backward ran (T_alt dense tiles, no tables)
    const int* slots;   // [B][T][Np] of the separable backward
    const long long* offsets;  // [B T + 1]: the tiles' first records in its compact partial array
    const int* overflow;       // [0] set where that array was too small, [1] the stamp of the tables
    int stamp;                 // tables_stamp of this call
    SuperSlots sup;
    int Np, N, C, Cp;   // C: channels of the caller's rows (feature kind), Cp: of the records
    const float *p0, *p1, *p2, *alphas;  // cov_inv_* | scales, rotations | gs_feature
    float eps;
    float *g_pos, *g0, *g1, *g2, *g_alpha, *g_col;  // feature kind: g_pos = d gs_feature
};

// One bit per lane of the caller's group.
__device__ __forceinline__ unsigned int group_ballot(bool p) {
    const unsigned long long m = __ballot(p) >> (threadIdx.x & (64 - kFinGroup));
    return kFinGroup == 32 ? (unsigned int)m : (unsigned int)m & ((1u << (kFinGroup % 32)) - 1u);
}

// Lane `lane` of a group adds, to its sums of fields lane, lane + kFinGroup, .., the records of
// Gaussian n in up to kFinGroup tiles: this lane's tile is `t` (`in`: it exists), in ascending lane
// order.  Group-uniform control flow; the other groups of the wave may be elsewhere.
__device__ __forceinline__ void group_add_tiles(const float* __restrict__ part, const int* __restrict__ slots,
                                                const long long* __restrict__ toff,
                                                int Np, int N, int NF, int n, int lane, int t, bool in,
                                                float (&acc)[kFinGroupFields]) {
    const int col = in ? slots[(size_t)t * Np + n] : -1;
    unsigned int tm = group_ballot(col >= 0);
    // where this lane's tile keeps the Gaussian's record (in floats; the lanes that read it fetch the two halves)
    const unsigned long long at = col >= 0 ? (unsigned long long)(toff[t] + col) * NF : 0ull;
    const int at_lo = (int)(unsigned int)at, at_hi = (int)(at >> 32);
    while (tm) {
        float val[kFinGroupAhead][kFinGroupFields];
#pragma unroll
        for (int u = 0; u < kFinGroupAhead; ++u) {
            const bool have = tm != 0u;
            const int src = have ? __builtin_ctz(tm) : 0;
            tm &= tm - 1u;  // (0 stays 0)
            const unsigned int lo = (unsigned int)__shfl(at_lo, src, kFinGroup);
            const unsigned int hi = (unsigned int)__shfl(at_hi, src, kFinGroup);
            const float* rec = part + (((unsigned long long)hi << 32) | lo);
#pragma unroll
            for (int v = 0; v < kFinGroupFields; ++v)
                val[u][v] = (have && lane + v * kFinGroup < NF) ? rec[lane + v * kFinGroup] : 0.0f;
        }
#pragma unroll
        for (int u = 0; u < kFinGroupAhead; ++u)
#pragma unroll
            for (int v = 0; v < kFinGroupFields; ++v) acc[v] += val[u][v];
    }
}

// All records of Gaussian n after a two-level binning: the listed super-tiles in ascending order,
// the tiles of each row-major.
__device__ __forceinline__ void group_sum_listed(const float* __restrict__ part, const int* __restrict__ slots,
                                                 const long long* __restrict__ toff,
                                                 const SuperSlots sup, int Np, int N, int NF, int n, int lane,
                                                 float (&acc)[kFinGroupFields]) {
    for (int s0 = 0; s0 < sup.stiles; s0 += kFinGroup) {
        const int stl = s0 + lane;
        unsigned int sm = group_ballot(stl < sup.stiles && sup.cslots[(size_t)stl * Np + n] >= 0);
        while (sm) {
            const int st = s0 + __builtin_ctz(sm);
            sm &= sm - 1;
            const int sy = st / sup.stiles_x, sx = st - sy * sup.stiles_x;
            for (int j0 = 0; j0 < kSuperX * kSuperY; j0 += kFinGroup) {
                const int j = j0 + lane;
                const int ty = sy * kSuperY + j / kSuperX, tx = sx * kSuperX + j % kSuperX;
                group_add_tiles(part, slots, toff, Np, N, NF, n, lane, ty * sup.tiles_x + tx,
                                j < kSuperX * kSuperY && ty < sup.tiles_y && tx < sup.tiles_x, acc);
            }
        }
    }
}

// After a one-level binning: the T tiles in ascending order.
__device__ __forceinline__ void group_sum_tiles(const float* __restrict__ part, const int* __restrict__ slots,
                                                const long long* __restrict__ toff,
                                                int T, int Np, int N, int NF, int n, int lane,
                                                float (&acc)[kFinGroupFields]) {
    for (int t0 = 0; t0 < T; t0 += kFinGroup)
        group_add_tiles(part, slots, toff, Np, N, NF, n, lane, t0 + lane, t0 + lane < T, acc);
}

// The same over the dense partials of the general backward (every tile holds column n).
__device__ __forceinline__ void group_sum_dense(const float* __restrict__ part, int T, int N, int NF, int n,
                                                int lane, float (&acc)[kFinGroupFields]) {
    for (int t0 = 0; t0 < T; t0 += kFinGroupAhead) {
        float val[kFinGroupAhead][kFinGroupFields];
#pragma unroll
        for (int u = 0; u < kFinGroupAhead; ++u)
#pragma unroll
            for (int v = 0; v < kFinGroupFields; ++v)
                val[u][v] = (t0 + u < T && lane + v * kFinGroup < NF)
                                ? part[((size_t)(t0 + u) * N + n) * NF + lane + v * kFinGroup] : 0.0f;
#pragma unroll
        for (int u = 0; u < kFinGroupAhead; ++u)
#pragma unroll
            for (int v = 0; v < kFinGroupFields; ++v) acc[v] += val[u][v];
    }
}

// kKind: 0 = operator level (cov_inv), 1 = function level (scales, rotations), 2 = module head (gs_feature)
template <int kKind>
__global__ __launch_bounds__(kThreads) void k_bwd_finalize_listed(const FinalizeArgs a) {
    __shared__ float mom[kFinGroupBatch][6];
    constexpr int kGroups = kThreads / kFinGroup;
    static_assert(kFinGroupBatch % kGroups == 0, "every group takes the same number of Gaussians");
    const int lane = threadIdx.x % kFinGroup, group = threadIdx.x / kFinGroup;
    const int b = blockIdx.y, n0 = blockIdx.x * kFinGroupBatch;
    const bool general = a.slots == nullptr || (a.flag != nullptr && *a.flag == 0);
    const int T = general ? a.T_alt : a.T;
    const int NF = 6 + a.Cp;
    const float* part = general ? a.partial + (size_t)b * T * NF * a.N : a.partial;
    const int* slots = a.slots != nullptr ? a.slots + (size_t)b * a.T * a.Np : nullptr;
    const long long* toff = general ? nullptr : a.offsets + (size_t)b * a.T;
    const bool lost = !general && (a.overflow[0] != 0 || a.overflow[1] != a.stamp);  // no gradient is known
    SuperSlots sup = a.sup;
    if (sup.cslots != nullptr) sup.cslots += (size_t)b * sup.stiles * a.Np;
    for (int k = 0; k < kFinGroupBatch / kGroups; ++k) {
        const int ln = k * kGroups + group;  // the groups work on neighbouring Gaussians at any time
        const int n = n0 + ln;
        if (n >= a.N) continue;  // group-uniform
        float acc[kFinGroupFields];
#pragma unroll
        for (int v = 0; v < kFinGroupFields; ++v) acc[v] = 0.0f;
        if (lost) {
#pragma unroll
            for (int v = 0; v < kFinGroupFields; ++v) acc[v] = __builtin_nanf("");
        } else if (general)
            group_sum_dense(part, T, a.N, NF, n, lane, acc);
        else if (a.sup.cslots != nullptr)
            group_sum_listed(part, slots, toff, sup, a.Np, a.N, NF, n, lane, acc);
        else
            group_sum_tiles(part, slots, toff, T, a.Np, a.N, NF, n, lane, acc);
        const size_t i = (size_t)b * a.N + n;
#pragma unroll
        for (int v = 0; v < kFinGroupFields; ++v) {
            const int f = lane + v * kFinGroup;  // this lane's field
            if (f < 6) {
                mom[ln][f] = acc[v];
            } else if (kKind == 2) {
                if (f < 6 + a.C) a.g_pos[i * (6 + a.C) + f] = acc[v];
            } else if (a.g_col != nullptr && f < NF) {
                a.g_col[i * a.Cp + f - 6] = a.alphas[i] * acc[v];
            }
        }
    }
    __syncthreads();
    const int n = n0 + threadIdx.x;
    if (threadIdx.x < kFinGroupBatch && n < a.N) {
        const size_t i = (size_t)b * a.N + n;
        if (kKind == 2)
            finalize_feature_geometry(mom[threadIdx.x], a.p0 + i * (6 + a.C), a.eps, a.g_pos + i * (6 + a.C));
        else
            finalize_geometry<kKind == 1>(mom[threadIdx.x], i, a.p0, a.p1, a.p2, a.alphas, a.eps, a.g_pos, a.g0, a.g1,
                                          a.g2, a.g_alpha);
    }
}

template <int kKind>
static void launch_finalize_listed(const FinalizeArgs& a, int B, hipStream_t stream) {
    hipLaunchKernelGGL(k_bwd_finalize_listed<kKind>, dim3((a.N + kFinGroupBatch - 1) / kFinGroupBatch, B),
                       dim3(kThreads), 0, stream, a);
}
