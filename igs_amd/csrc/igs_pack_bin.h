// igs_pack_bin.h -- pack kernels (records + bin records) and the per-tile Gaussian lists (k_bin).
// Included by igs_gs2d.hip inside its anonymous namespace (one translation unit).
#pragma once

// ----------------------------------------------------------------------------- pack
// Reach box of a Gaussian: the axis-aligned bounding box of the ellipse q <= Q, outside of which
// the kernels skip it.  Q comes from the skip limit L of the call (in units of the kernels'
// exponent q' = -0.5 log2(e) q, so that e = 2^q'):
//   * L = kExactLimit (skip weight 0): the box bounds q' >= -160, ten binades under the -149/-150
//     at which exp2 returns 0 in fp32 whatever the denormal mode (the margin covers the rounding of
//     q' itself, which is a few ulp of its largest term).  Pixels outside the box receive exactly +0
//     from this Gaussian and give exactly 0 to its gradient sums, so skipping them changes no bit.
//   * L < kExactLimit (skip weight w > 0, L = -log2 w): a pair is skipped only where
//     e < w / max(1, |alpha|), i.e. where both the weight alpha e and the bare exponential (which is
//     what the gradient of alpha sums) are below w.  The limit of Gaussian n is
//     L_n = min(kExactLimit, L + log2 max(1, |alpha_n|)).
//   The boxes are made for the call's skip weight; k_bin may leave out heavier Gaussians for a
//   tile (as far as the tile's allowance goes, see k_bin), which only removes more of what the box
//   lets through.
// The box is five binades wider than the tile test of k_bin (ellipse_reaches), as in the exact case.
// Half extents: sqrt(Q Sigma_xx), sqrt(Q Sigma_yy) with Sigma the covariance that (A, B, D) invert.
// A record with a non-finite field or a non-positive-definite (A, B, D) gets an unbounded box (its
// NaN/inf must propagate as without culling); padding records get an empty one.
//
// What k_bin needs of a Gaussian sits in a "bin record" of its own, 8 floats, so that the binning
// reads one contiguous stream instead of a box and then, for the boxes that meet the tile, the
// Gaussian's record: (px, py, hx, hy) = centre and half extents of the box (+inf: unbounded, -inf:
// empty) and (a, b2, d, alpha) = the quadratic form of -q' (the negated A', B2', D' of the record).
// The bin records [B][Np] follow the records in the packed buffer.
constexpr float kExactLimit = 155.0f;
constexpr double kHalfLog2e = 0.72134752044448170368;

// limit of one Gaussian from the call's limit and its alpha (finite alpha)
__device__ __forceinline__ float skip_limit(float limit, float alpha) {
    return fminf(kExactLimit, limit + __log2f(fmaxf(1.0f, fabsf(alpha))));
}

// half extents (hx, hy) of the reach box
__device__ __forceinline__ float2 reach_extent(float px, float py, double sxx, double syy, bool bounded,
                                               float limit_n) {
    const float inf = __builtin_inff();
    if (!bounded || !(sxx >= 0.0) || !(syy >= 0.0) || !isfinite(px) || !isfinite(py)) return make_float2(inf, inf);
    const double Q = ((double)limit_n + 5.0) / kHalfLog2e;
    // rounded outwards: one part in 1e5 is far more than the fp32 rounding of the bounds px -+ hx
    const double hx = sqrt(Q * sxx) * 1.00001, hy = sqrt(Q * syy) * 1.00001;
    const double ax = fabs((double)px) * 1e-6 + 1e-30, ay = fabs((double)py) * 1e-6 + 1e-30;
    return make_float2((float)(hx + ax), (float)(hy + ay));
}

__device__ __forceinline__ void write_bin_record(float4* bins, size_t i, float px, float py, float2 h,
                                                 float A, float B2, float D, float alpha) {
    bins[2 * i] = make_float4(px, py, h.x, h.y);
    bins[2 * i + 1] = make_float4(-A, -B2, -D, alpha);
}
__device__ __forceinline__ void write_empty_bin_record(float4* bins, size_t i) {
    const float inf = __builtin_inff();
    bins[2 * i] = make_float4(0.0f, 0.0f, -inf, -inf);
    bins[2 * i + 1] = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
}

// The call's skip limit and skip fraction travel behind the bin records in the packed buffer
// (4 floats, the first two used), where k_bin reads them: the forward and the backward then need no
// argument for them.  Behind them sits one all-zero record (kZeroRecFloats floats, the widest
// record), which the forward's direct global-to-LDS loads read for the slots past a list's end.
constexpr int kZeroRecFloats = 28;
__device__ __forceinline__ void write_skip_limit(float4* bins, int B, int Np, float limit, float fraction) {
    float4* tail = bins + (size_t)2 * B * Np;
    tail[0] = make_float4(fminf(limit, kExactLimit), fraction, 0.0f, 0.0f);
    for (int i = 0; i < kZeroRecFloats / 4; ++i) tail[1 + i] = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
}

// Records of the separable kernels.  With a positive definite form the square can be completed,
//   q' = A'dx^2 + B2'dx dy + D'dy^2 = -(sD dy + skD dx)^2 + A''dx^2      (forward: rows inside a column)
//                                    = -(sA dx + skA dy)^2 + D''dy^2      (backward: columns inside a row)
// with sD = sqrt(-D'), skD = -B2' / (2 sD), A'' = A' - B2'^2 / (4 D') = k det / D (k = -0.5 log2 e) and
// the same with A and D exchanged: one term per pair instead of two, the other hoisted, and both terms
// are non-positive, so nothing cancels however long and tilted the ellipse is.  The six values are
// formed in fp64 from the unrounded A, B, D (A'' and D'' from the determinant: the difference
// A' - B2'^2 / (4 D') of the rounded values would lose the digits that a thin ellipse needs).
// A record whose form is not positive definite, or has a non-finite value anywhere, is tagged (forward
// record: NaN in place of a copy of sD, which a single comparison with the wave's limit on sD turns into
// the choice of the evaluation; backward record: 1 in place of 0): the kernels evaluate it term by term
// as on general grids, from A', B2', D', which the forward record carries as well.
struct SepTerms {
    float sD, skD, A2, sA, skA, D2;
    bool regular;
};
__device__ __forceinline__ SepTerms sep_terms(double A, double Bc, double D, double det, bool finite_record) {
    constexpr double k = -0.72134752044448170368;
    SepTerms t;
    const double sD = sqrt(-k * D), sA = sqrt(-k * A);
    t.sD = (float)sD;
    t.skD = (float)(-k * Bc / sD);
    t.A2 = (float)(k * det / D);
    t.sA = (float)sA;
    t.skA = (float)(-k * Bc / sA);
    t.D2 = (float)(k * det / A);
    t.regular = finite_record && A > 0.0 && D > 0.0 && det > 0.0 && isfinite(t.sD) && isfinite(t.skD) &&
                isfinite(t.A2) && isfinite(t.sA) && isfinite(t.skA) && isfinite(t.D2) && t.sD > 0.0f && t.sA > 0.0f;
    return t;
}
__device__ __forceinline__ void write_brec(float4* brec, size_t i, const SepTerms& t) {
    brec[i] = t.regular ? make_float4(t.sA, t.skA, t.D2, 0.0f) : make_float4(0.0f, 0.0f, 0.0f, 1.0f);
}

// Stores the records of one Gaussian from registers: `rec` holds the plain record (px, py, A', B2', D',
// alpha, alpha*c_0..C-1, zeros behind); every index is a compile-time constant after unrolling, and a
// lane writes float4s.  The plain record also gets the y range of the reach box where it has two spare
// floats; the forward record of the separable kernels (RSF > 0) is the same with the completed square in
// place of A', B2', D', and behind the colours the tag and A', B2', D'.
__device__ __forceinline__ void store_records(float (&rec)[kZeroRecFloats], int C, int RS, int RSF, float py, float2 ext,
                                              const SepTerms& t, float* __restrict__ r, float* __restrict__ fr) {
    const float Ap = rec[2], B2p = rec[3], Dp = rec[4];
    if (RS >= 8 + C) {  // room in the record: the y range of the box travels with it
#pragma unroll
        for (int c = 6; c < kZeroRecFloats - 1; ++c)
            if (c == 6 + C) {
                rec[c] = py - ext.y;
                rec[c + 1] = py + ext.y;
            }
    }
    float4* r4 = reinterpret_cast<float4*>(r);  // records are 4 k floats apart behind a 16-byte aligned base
#pragma unroll
    for (int q = 0; q < kZeroRecFloats / 4; ++q)
        if (4 * q < RS) r4[q] = make_float4(rec[4 * q], rec[4 * q + 1], rec[4 * q + 2], rec[4 * q + 3]);
    if (RSF == 0) return;
    rec[2] = t.sD;
    rec[3] = t.skD;
    rec[4] = t.A2;
#pragma unroll
    for (int c = 6; c < kZeroRecFloats - 5; ++c)
        if (c == 6 + C) {
            rec[c] = t.regular ? t.sD : __builtin_nanf("");
            rec[c + 1] = Ap;
            rec[c + 2] = B2p;
            rec[c + 3] = Dp;
            rec[c + 4] = 0.0f;
            rec[c + 5] = 0.0f;
        }
    float4* f4 = reinterpret_cast<float4*>(fr);
#pragma unroll
    for (int q = 0; q < kZeroRecFloats / 4; ++q)
        if (4 * q < RSF) f4[q] = make_float4(rec[4 * q], rec[4 * q + 1], rec[4 * q + 2], rec[4 * q + 3]);
}

// One thread per record.  Record: px, py, A', B2', D', alpha, alpha*c_0.. (padded to x4)
// with A' = k A, B2' = 2 k B, D' = k D, k = -0.5 log2 e.  Records N..Np-1 are zero.
template <bool kScaleRot>
__global__ __launch_bounds__(kThreads) void k_pack(const float* __restrict__ position,
                                                   const float* __restrict__ p0,  // cov00 | scales
                                                   const float* __restrict__ p1,  // cov01 | rotations
                                                   const float* __restrict__ p2,  // cov11 | unused
                                                   const float* __restrict__ alphas,
                                                   const float* __restrict__ colors, int N,
                                                   int Np, int C, int RS, float eps,
                                                   float limit, float fraction,
                                                   float* __restrict__ packed,
                                                   float4* __restrict__ boxes,
                                                   float* __restrict__ frecs, int RSF,
                                                   float4* __restrict__ brecs) {
    const int n = blockIdx.x * kThreads + threadIdx.x;
    const int b = blockIdx.y;
    if (n == 0 && b == 0) write_skip_limit(boxes, gridDim.y, Np, limit, fraction);
    if (n >= Np) return;
    float* r = packed + ((size_t)b * Np + n) * RS;
    float* fr = frecs + ((size_t)b * Np + n) * RSF;
    if (n >= N) {  // padding: alpha = 0 and e = exp2(0) = 1, so it contributes exactly 0
        for (int c = 0; c < RS; ++c) r[c] = 0.0f;
        for (int c = 0; c < RSF; ++c) fr[c] = 0.0f;
        brecs[(size_t)b * Np + n] = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
        write_empty_bin_record(boxes, (size_t)b * Np + n);
        return;
    }
    const size_t i = (size_t)b * N + n;
    // The closed form runs in fp64 and is rounded once: an error of a few fp32 ulp in A', B2', D'
    // would be multiplied by |q| (tens, for sharp Gaussians) in the exponent.  O(BN) work.
    double A, Bc, D, sxx, syy, det;
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
        det = i0 * i1;
        bounded = v0 > 0.0 && v1 > 0.0;
    } else {
        A = p0[i];
        Bc = p1[i];
        D = p2[i];
        det = A * D - Bc * Bc;
        bounded = A > 0.0 && det > 0.0;
        sxx = D / det;
        syy = A / det;
    }
    constexpr double k = -0.72134752044448170368;  // -0.5 * log2(e)
    const float al = alphas[i];
    const float px = position[2 * i], py = position[2 * i + 1];
    // The record is put together in registers (every index below is a compile-time constant after
    // unrolling) and stored as float4s: the colour loads are then in flight together and a lane
    // writes RS / 4 times instead of RS times (C = 16, 131072 records: 39 -> 9 us).
    float rec[kZeroRecFloats];
#pragma unroll
    for (int c = 0; c < kZeroRecFloats; ++c) rec[c] = 0.0f;
    rec[0] = px;
    rec[1] = py;
    rec[2] = (float)(k * A);
    rec[3] = (float)(2.0 * k * Bc);
    rec[4] = (float)(k * D);
    rec[5] = al;
    bool fin = isfinite(al) && isfinite(rec[2]) && isfinite(rec[3]) && isfinite(rec[4]);
    float col[IGS_MAX_CHANNELS];
#pragma unroll
    for (int c = 0; c < IGS_MAX_CHANNELS; ++c) col[c] = c < C ? colors[i * C + c] : 0.0f;
#pragma unroll
    for (int c = 0; c < IGS_MAX_CHANNELS; ++c) {
        const float v = al * col[c];
        if (c < C) {
            rec[6 + c] = v;
            fin = fin && isfinite(v) && isfinite(col[c]);
        }
    }
    const float2 ext = reach_extent(px, py, sxx, syy, bounded && fin, skip_limit(limit, al));
    write_bin_record(boxes, (size_t)b * Np + n, px, py, ext, rec[2], rec[3], rec[4], al);
    const SepTerms t = sep_terms(A, Bc, D, det, bounded && fin && isfinite(px) && isfinite(py));
    write_brec(brecs, (size_t)b * Np + n, t);
    store_records(rec, C, RS, RSF, py, ext, t, r, fr);
}

// Module head fused into the pack: reads gs_feature rows [px, py, log_s0, log_s1, theta,
// opacity logit (unused), c_0..c_{C-1}] (reference src/igs/gs2d.py:635-644) and applies the
// module's activations scales = exp(log_s) + eps, alpha = 1 (src/igs/gs2d.py:673-675), plus
// an optional position offset (pos_map_offset, src/igs/gs2d.py:654-667).  Also writes the raw
// colours [B][N][Cp] (zero-padded to the kernels' channel count) that the backward reads.
__global__ __launch_bounds__(kThreads) void k_pack_feature(const float* __restrict__ feat,
                                                           const float* __restrict__ pos_off, int N,
                                                           int Np, int C, int Cp, int RS, float eps,
                                                           float limit, float fraction,
                                                           float* __restrict__ packed,
                                                           float4* __restrict__ boxes,
                                                           float* __restrict__ frecs, int RSF,
                                                           float4* __restrict__ brecs,
                                                           float* __restrict__ colors_out) {
    const int n = blockIdx.x * kThreads + threadIdx.x;
    const int b = blockIdx.y;
    if (n == 0 && b == 0) write_skip_limit(boxes, gridDim.y, Np, limit, fraction);
    if (n >= Np) return;
    float* r = packed + ((size_t)b * Np + n) * RS;
    float* fr = frecs + ((size_t)b * Np + n) * RSF;
    if (n >= N) {
        for (int c = 0; c < RS; ++c) r[c] = 0.0f;
        for (int c = 0; c < RSF; ++c) fr[c] = 0.0f;
        brecs[(size_t)b * Np + n] = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
        write_empty_bin_record(boxes, (size_t)b * Np + n);
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
    float rec[kZeroRecFloats];
#pragma unroll
    for (int c = 0; c < kZeroRecFloats; ++c) rec[c] = 0.0f;
    rec[0] = px;
    rec[1] = py;
    rec[2] = (float)(k * A);
    rec[3] = (float)(2.0 * k * Bc);
    rec[4] = (float)(k * D);
    rec[5] = 1.0f;
    bool fin = isfinite(rec[2]) && isfinite(rec[3]) && isfinite(rec[4]);
#pragma unroll
    for (int c = 0; c < IGS_MAX_CHANNELS; ++c) {
        const float col = c < C ? f[6 + c] : 0.0f;
        rec[6 + c] = col;
        if (c < Cp) colors_out[i * Cp + c] = col;
        fin = fin && isfinite(col);
    }
    const bool bounded = fin && v0 > 0.0 && v1 > 0.0;
    const float2 ext = reach_extent(px, py, cs * cs * v0 + sn * sn * v1, sn * sn * v0 + cs * cs * v1, bounded,
                                    skip_limit(limit, 1.0f));
    write_bin_record(boxes, (size_t)b * Np + n, px, py, ext, rec[2], rec[3], rec[4], 1.0f);
    const SepTerms t = sep_terms(A, Bc, D, i0 * i1, bounded && isfinite(px) && isfinite(py));
    write_brec(brecs, (size_t)b * Np + n, t);
    store_records(rec, Cp, RS, RSF, py, ext, t, r, fr);
}

// ----------------------------------------------------------------------------- binning
// Per pixel tile, the Gaussians whose reach box meets the tile's coordinate range and whose
// ellipse can reach it (ellipse_reaches), as a list of indices in increasing order (so that
// sums over a list keep the order of the unculled sum), and the count.  One workgroup per
// (tile, image) scans all N boxes — or, in a two-level binning, a chunk of them for a super-tile
// (first level) or the segments of its super-tile's list (second level); positions come from
// ballots and a fixed-order prefix over the waves, so the lists are reproducible.
// With `slots` set, the inverse map is written as well: slots[b][tile][n] = position of
// Gaussian n in the tile's list, or -1 when it is not listed; written for every candidate, i.e.
// every n < N except at the second level of a two-level binning, where a tile's entries exist
// only for the Gaussians listed for its super-tile (whose table, non-negative = listed, the
// first level writes).
// Separable grids only: a tile is tile_w columns x tile_h rows and its coordinate range is
// [min, max] of x over its columns and of y over its rows (no monotonicity assumed).
struct BinArgs {
    const float4* bins;   // [B][Np][2] bin records
    const float* x;
    const float* y;
    long sxb, sxw, syb, syh;
    int N, Np, H, W;
    int tile_w, tile_h, tiles_x, tiles_y;
    int* counts;  // [B][tiles] ([B][tiles][K] with chunks)
    int* lists;   // [B][tiles][Np]
    int* slots;   // [B][tiles][Np] or nullptr
    // Two-level binning.  First level (chunk > 0): the tiles are super-tiles of kSuperX x kSuperY
    // tiles and gridDim.y = K workgroups share a super-tile, workgroup k scanning the Gaussians
    // [k chunk, (k + 1) chunk) into segment k of the list (at offset k chunk, with its own count).
    // Second level (cand_lists set): a tile scans the K segments of its super-tile's list, in order,
    // instead of all N Gaussians.
    int chunk;
    const int* cand_counts;  // [B][stiles][cand_K]
    const int* cand_lists;   // [B][stiles][Np], segment k at offset k cand_chunk
    int cand_K, cand_chunk, stiles_x, stiles;
    const float* limit;  // the call's skip limit and fraction, written by the pack kernel behind the bin records
    const int* flag;
    int want;
    int no_cull;  // list every candidate (IGS_OPT_NO_CULL): the reference point for "culling changes no bit"
    // Four lists per tile (the forward's wave lists; sub_nx = 0: one list).  The tile is sub_nx x
    // (4 / sub_nx) rectangles of sub_w columns x sub_h rows (rectangle w: column block w % sub_nx, row
    // block w / sub_nx), each with a list of its own; the image's lists are numbered by rectangle,
    // row after row of rectangles.
    int sub_nx, sub_w, sub_h;
    // Where the numbering of `counts` and `lists` is not the launch's own (one list per tile, row
    // after row of tiles_x tiles): lists per image and lists per row.  0: the launch's own.
    int img_lists, row_lists;
    // The launch carries dynamic LDS for one byte (four with four lists) per candidate, in which the
    // scan that settles what the tile skips leaves each candidate's weight class for the scan that
    // lists; 0: that scan evaluates the rectangle test again.
    int store_classes;
};

// Tiles per super-tile of the two-level binning (each way) and the most segments per list.
constexpr int kSuperX = 4, kSuperY = 4, kBinMaxChunks = 64;

constexpr int kBinThreads = 1024, kBinWaves = kBinThreads / 64;  // many loads in flight per tile
// With four lists per tile a lane holds four rectangles' worth of intermediate values: at 1024 threads
// (128 registers per lane) a third of them spilled to scratch memory.
#ifndef IGS_BIN_THREADS_MASKS
#define IGS_BIN_THREADS_MASKS 512
#endif
constexpr int kBinThreadsMasks = IGS_BIN_THREADS_MASKS;

// Second test for a Gaussian whose reach box meets the tile: can its ellipse reach the tile's
// coordinate rectangle at all (the box of a long, rotated ellipse is mostly empty), and with what
// weight at most?  With P = -q' = a dx^2 + b2 dx dy + d dy^2 (a, b2, d = -A', -B2', -D' of the
// record), the minimum of P over the rectangle is 0 when it holds the centre and else lies on an
// edge, where P is a parabola in one variable.  The kernels' weight is exactly 0 where their fp32 q'
// is below -150; both their q' and the P evaluated here differ from the exact value by a few ulp of
// the largest term, bounded over the rectangle by T below.  reach_p returns min P - 4e-6 T: every
// weight of the Gaussian on the rectangle is at most 2^-reach_p, and exactly 0 in the kernels where
// reach_p > kExactLimit (the same margin against rounding as the reach box has, so dropping such a
// tile changes no bit).  -inf (never dropped) when the rectangle holds the centre or the form is
// not safely positive definite; NaN for a NaN record, which fails every comparison and stays listed.
// Evaluated twice per candidate (for the tile's histogram and for the verdict): without contraction
// of multiplies and adds, so that both evaluations are the same arithmetic and agree bit for bit.
__device__ __forceinline__ float reach_form(float a, float b2, float d, float x, float y) {
#pragma clang fp contract(off)
    return fmaf(fmaf(b2, x, d * y), y, (a * x) * x);
}
__device__ __forceinline__ float reach_p(float4 q0, float4 q1, float txlo, float txhi, float tylo, float tyhi) {
#pragma clang fp contract(off)
    const float a = q1.x, b2 = q1.y, d = q1.z;
    const float x0 = txlo - q0.x, x1 = txhi - q0.x, y0 = tylo - q0.y, y1 = tyhi - q0.y;
    // straight-line code (every path is taken by some lane of a wave anyway)
    const bool inside = x0 <= 0.0f && x1 >= 0.0f && y0 <= 0.0f && y1 >= 0.0f;
    // the argument below needs a form that is positive definite beyond the rounding of its
    // (fp32) coefficients; ellipses thinner than about 1:600 simply stay listed
    const bool definite = a > 0.0f && (4.0f * a) * d - b2 * b2 > (4e-5f * a) * d;
    // Only the edges that face the centre can hold the minimum: P grows along every ray from the
    // centre, and the ray to a point of the rectangle enters it through such an edge.  The vertex
    // of an edge's parabola uses the hardware reciprocal (its error is of second order in P).
    const float inf = __builtin_inff();
    const bool vx = x0 > 0.0f || x1 < 0.0f, vy = y0 > 0.0f || y1 < 0.0f;
    const float xe = x0 > 0.0f ? x0 : x1, ye = y0 > 0.0f ? y0 : y1;
    const float ky = (-0.5f * b2) * __builtin_amdgcn_rcpf(d), kx = (-0.5f * b2) * __builtin_amdgcn_rcpf(a);
    const float pv = vx ? reach_form(a, b2, d, xe, fminf(fmaxf(ky * xe, y0), y1)) : inf;
    const float ph = vy ? reach_form(a, b2, d, fminf(fmaxf(kx * ye, x0), x1), ye) : inf;
    const float pmin = fminf(pv, ph);
    const float mx = fmaxf(fabsf(x0), fabsf(x1)), my = fmaxf(fabsf(y0), fabsf(y1));
    const float T = ((a * mx) * mx + (fabsf(b2) * mx) * my) + (d * my) * my;
    const float p = pmin - 4e-6f * T;
    return (inside || !definite) ? -inf : p;
}

// The weight classes of the binning: class k holds the (Gaussian, tile) pairs whose largest term of
// a denominator, e max(1, |alpha|) <= 2^-(reach_p - log2 max(1, |alpha|)), lies in
// (2^-((k + 1) / kBinRes), 2^-(k / kBinRes)].  -1: not classed (the bound exceeds 1, or NaN) and
// never skipped.
constexpr int kBinRes = 2;
constexpr int kMaxSkipClasses = 253;  // (a class relative to the call's fits a byte)
constexpr int kBinClasses = 320;  // >= kExactLimit kBinRes + 1, a multiple of 64
static_assert(kBinClasses >= (int)kExactLimit * kBinRes + 1 && kBinClasses % 64 == 0, "weight classes");
__device__ __forceinline__ int weight_class(float p, float alpha) {
#pragma clang fp contract(off)
    const float r = (p - __log2f(fmaxf(1.0f, fabsf(alpha)))) * (float)kBinRes;
    return r >= 0.0f ? (int)fminf(r, (float)(kBinClasses - 1)) : -1;
}
// first class that the call's skip limit L (weights below 2^-L are skipped) lets skip entirely
__device__ __forceinline__ int base_class(float limit) {
    return limit < kExactLimit ? (int)ceilf(limit * (float)kBinRes) : 0x7fffffff;
}
// verdict for one rectangle: skipped when the weight is exactly zero there, or its class is one of
// those the tile skips
__device__ __forceinline__ bool ellipse_reaches(float4 q0, float4 q1, float txlo, float txhi, float tylo,
                                                float tyhi, int first_skipped) {
    const float p = reach_p(q0, q1, txlo, txhi, tylo, tyhi);
    return !(p > kExactLimit || weight_class(p, q1.w) >= first_skipped);
}

// A Gaussian's smallest weight over the tile's coordinate rectangle: alpha 2^(-max P), P = -q' being
// convex, its maximum over the rectangle is at a corner.  Summed over Gaussians with alpha >= 0 this
// bounds every denominator of the tile from below.  Rounded down by 1e-3 against the fp32 rounding
// of P at the corners (a few 1e-6 of its largest term, which matters only while 2^-P does).
__device__ __forceinline__ float least_weight(float4 q0, float4 q1, float txlo, float txhi, float tylo,
                                              float tyhi) {
    const float a = q1.x, b2 = q1.y, d = q1.z;
    const float x0 = txlo - q0.x, x1 = txhi - q0.x, y0 = tylo - q0.y, y1 = tyhi - q0.y;
    auto form = [&](float x, float y) { return fmaf(fmaf(b2, x, d * y), y, a * x * x); };
    const float pmax = fmaxf(fmaxf(form(x0, y0), form(x0, y1)), fmaxf(form(x1, y0), form(x1, y1)));
    const float w = q1.w * hw_exp2(-pmax) * 0.999f;
    return w > 0.0f ? w : 0.0f;  // NaN, inf - inf and the like count as nothing
}

// (the body of k_bin for tile `t` of a's launch: also called by k_bin_pair, one launch for two sets of lists)
template <bool kMasks>
__device__ __forceinline__ void bin_tile(const BinArgs& a, const int t) {
    if (a.flag != nullptr && *a.flag != a.want) return;
    __shared__ float red[4][kBinWaves];
    __shared__ int wsum[kMasks ? 4 : 1][kBinWaves];
    __shared__ int seg_first[kBinMaxChunks + 1];  // second level: first candidate index of each segment
    __shared__ int hist[kMasks ? 4 : 1][kBinClasses];  // candidates per weight class and list
    __shared__ int first_skipped_s[kMasks ? 4 : 1];
    extern __shared__ unsigned int class_store[];  // per candidate: kbase - class per list, 0 = skipped, 255 = listed
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    for (int i = tid; i < (kMasks ? 4 : 1) * kBinClasses; i += blockDim.x) (&hist[0][0])[i] = 0;
    // launched with 256 to kBinThreads threads (bin_threads): the reductions below run over kBinWaves
    // slots, those of waves that do not exist hold the neutral element
    const int nthreads = blockDim.x, nwaves = nthreads >> 6;
    if (tid < kBinWaves && tid >= nwaves) {
#pragma unroll
        for (int f = 0; f < 4; ++f) red[f][tid] = __builtin_inff();
#pragma unroll
        for (int l = 0; l < (kMasks ? 4 : 1); ++l) wsum[l][tid] = 0;
    }
    const int tiles = a.tiles_x * a.tiles_y;
    const int kc = blockIdx.y, K = gridDim.y, b = blockIdx.z;
    const int ty = t / a.tiles_x, tx = t - ty * a.tiles_x;
    const int c0 = tx * a.tile_w, c1 = min(a.W, c0 + a.tile_w);
    const int r0 = ty * a.tile_h, r1 = min(a.H, r0 + a.tile_h);
    const float inf = __builtin_inff();
    const float4* bins = a.bins + (size_t)2 * b * a.Np;
    // The candidates, numbered 0..M-1: all Gaussians; or this workgroup's chunk of them (first
    // level); or the entries of the super-tile's list, segment after segment (second level).
    int first = 0, M = a.N;
    const int* cand = nullptr;
    if (a.chunk > 0) {
        first = kc * a.chunk;
        M = max(0, min(a.N, first + a.chunk) - first);
    }
    if (a.cand_lists != nullptr) {
        const size_t st = (size_t)b * a.stiles + (ty / kSuperY) * a.stiles_x + tx / kSuperX;
        cand = a.cand_lists + st * a.Np;
        if (tid == 0) {
            int run = 0;
            for (int j = 0; j < a.cand_K; ++j) {
                seg_first[j] = run;
                run += a.cand_counts[st * a.cand_K + j];
            }
            for (int j = a.cand_K; j <= kBinMaxChunks; ++j) seg_first[j] = run;
        }
        __syncthreads();
        M = seg_first[kBinMaxChunks];
    }
    // candidate index -> Gaussian index
    auto gaussian_of = [&](int i) {
        if (cand == nullptr) return first + i;
        int seg = 0;  // the last segment that starts at or before i (binary search over 64 entries)
#pragma unroll
        for (int step = kBinMaxChunks / 2; step > 0; step >>= 1)
            if (seg_first[seg + step] <= i) seg += step;
        return cand[(size_t)seg * a.cand_chunk + (i - seg_first[seg])];
    };
    // Each wave scans one contiguous share of the candidates, without barriers inside a scan: once
    // for what the tile may skip (skip fraction only), once to classify and count, and once
    // (from the kept verdicts, with the shares' counts prefixed in wave order) to write.
    const int per_wave = ((M + nwaves - 1) / nwaves + 63) & ~63;
    const int nb = wave * per_wave, ne = min(M, nb + per_wave);
    const unsigned long long below = (1ull << lane) - 1ull;
    // The bin records of kU candidates per lane are loaded together (2 kU loads in flight).  The
    // first batch of a wave is loaded before anything else, so that its latency overlaps with the
    // tile's coordinate range, and is kept for both scans: small problems never load twice.
    constexpr int kU = 4;
    struct Batch {
        int n[kU];
        float4 q0[kU], q1[kU];
    };
    auto load_batch = [&](int n0, Batch& bt) {
#pragma unroll
        for (int u = 0; u < kU; ++u) bt.n[u] = gaussian_of(min(n0 + u * 64 + lane, M - 1));  // M > 0 in the loops
#pragma unroll
        for (int u = 0; u < kU; ++u) {
            bt.q0[u] = bins[2 * bt.n[u]];
            bt.q1[u] = bins[2 * bt.n[u] + 1];
        }
    };
    Batch head;
#pragma unroll
    for (int u = 0; u < kU; ++u) {
        head.n[u] = 0;
        head.q0[u] = head.q1[u] = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
    }
    if (nb < ne) load_batch(nb, head);

    float xlo = inf, xhi = -inf, ylo = inf, yhi = -inf;
    bool bad = false;
    constexpr bool masks = kMasks;  // a.sub_nx > 0
    if (!masks) {
        for (int c = c0 + tid; c < c1; c += nthreads) {
            const float v = a.x[b * a.sxb + (long)c * a.sxw];
            bad = bad || !(v == v);
            xlo = fminf(xlo, v);
            xhi = fmaxf(xhi, v);
        }
        for (int r = r0 + tid; r < r1; r += nthreads) {
            const float v = a.y[b * a.syb + (long)r * a.syh];
            bad = bad || !(v == v);
            ylo = fminf(ylo, v);
            yhi = fmaxf(yhi, v);
        }
    } else if (wave < 4) {  // wave w takes the rectangle of the forward's wave w: its range is this wave's result
        const int c = c0 + (wave % a.sub_nx) * a.sub_w + lane;
        const int r = r0 + (wave / a.sub_nx) * a.sub_h + lane;
        if (lane < a.sub_w && c < c1) {
            xlo = xhi = a.x[b * a.sxb + (long)c * a.sxw];
            bad = !(xlo == xlo);
        }
        if (lane < a.sub_h && r < r1) {
            ylo = yhi = a.y[b * a.syb + (long)r * a.syh];
            bad = bad || !(ylo == ylo);
        }
    }
    if (bad || a.no_cull) {  // a NaN coordinate, or culling switched off: nothing may be culled for this tile
        xlo = ylo = -inf;
        xhi = yhi = inf;
    }
    // minima of (xlo, -xhi, ylo, -yhi) over the workgroup: within each wave by lane exchanges, then
    // over the 16 waves' results through LDS (fminf drops NaN, which `bad` has already handled)
    float rv[4] = {xlo, -xhi, ylo, -yhi};
#pragma unroll
    for (int f = 0; f < 4; ++f)
#pragma unroll
        for (int k = 32; k > 0; k >>= 1) rv[f] = fminf(rv[f], __shfl_xor(rv[f], k));
    if (lane == 0)
#pragma unroll
        for (int f = 0; f < 4; ++f) red[f][wave] = rv[f];
    __syncthreads();
#pragma unroll
    for (int f = 0; f < 4; ++f) {
        rv[f] = red[f][lane & (kBinWaves - 1)];
#pragma unroll
        for (int k = kBinWaves / 2; k > 0; k >>= 1) rv[f] = fminf(rv[f], __shfl_xor(rv[f], k));
    }
    const float txlo = rv[0], txhi = -rv[1], tylo = rv[2], tyhi = -rv[3];
    // the four waves' rectangles (xlo, xhi, ylo, yhi); one that is empty along an axis holds no pixel
    float sub[4][4];
    bool sub_any[4];
#pragma unroll
    for (int w = 0; w < 4; ++w) {
        sub[w][0] = masks ? red[0][w] : 0.0f;
        sub[w][1] = masks ? -red[1][w] : 0.0f;
        sub[w][2] = masks ? red[2][w] : 0.0f;
        sub[w][3] = masks ? -red[3][w] : 0.0f;
        sub_any[w] = sub[w][0] <= sub[w][1] && sub[w][2] <= sub[w][3];
    }
    const float limit = a.limit[0];
    const float fraction = a.limit[1];
    // The image's lists are numbered by tile; with four lists per tile by rectangle, row after row of
    // rectangles (rectangle l of the tile lies in row (4 / sub_nx) ty + l / sub_nx and column
    // sub_nx tx + l % sub_nx): the numbering that a binning with one workgroup per rectangle gives
    // (which then sets img_lists and row_lists, rectangles outside the image having no workgroup).
    const size_t img_first = (size_t)b * (a.img_lists > 0 ? a.img_lists : tiles * (masks ? 4 : 1));
    const int row_lists = a.row_lists > 0 ? a.row_lists : a.tiles_x * (masks ? a.sub_nx : 1);
    auto list_no = [&](int l) {
        return img_first + (masks ? (size_t)(ty * (4 / a.sub_nx) + l / a.sub_nx) * row_lists + tx * a.sub_nx + l % a.sub_nx
                                  : (size_t)ty * row_lists + tx);
    };
    int* list = a.lists + list_no(0) * a.Np + (size_t)kc * a.chunk;
    int* slot = a.slots ? a.slots + ((size_t)b * tiles + t) * a.Np : nullptr;
    // "definitely outside" negated, so that NaN bounds count as inside
    auto meets_tile = [&](const Batch& bt, int u) {
        return !(bt.q0[u].x + bt.q0[u].z < txlo || bt.q0[u].x - bt.q0[u].z > txhi ||
                 bt.q0[u].y + bt.q0[u].w < tylo || bt.q0[u].y - bt.q0[u].w > tyhi);
    };
    // What a tile may skip.  Every Gaussian that is not listed for a tile changes the tile's
    // denominators by at most its largest weight there, and the call allows N (w + f S) in total,
    // w = 2^-limit the skip weight, f the skip fraction and S a lower bound of the tile's
    // denominators (the sum of the least weights of the candidates whose box meets it; 0 if one of
    // them has a negative or non-finite alpha).  Classes from kbase on hold weights of at most w: they
    // are skipped, and so are the Gaussians that are no candidates here (their boxes miss the tile, or
    // the first level of a two-level binning dropped them: below w as well); with n the number of
    // classed candidates above w that leaves n w + N f S for them, which the lightest classes take up
    // as far as it goes, each candidate counted with the upper end of its class.
    // Not at the first level of a two-level binning (its lists must hold what any of its tiles may
    // list), nor where nothing is culled.
    const int kbase = base_class(limit);
    constexpr int kL = kMasks ? 4 : 1;  // lists per tile
    int first_skipped[kL];
#pragma unroll
    for (int l = 0; l < kL; ++l) first_skipped[l] = kbase;
    const bool settle = fraction > 0.0f && a.chunk == 0 && txlo > -inf && !a.no_cull;  // workgroup-uniform
    if (settle) {
        float sum = 0.0f;
        bool negative = false;
        int it = 0;
        for (int n0 = nb; n0 < ne; n0 += 64 * kU, ++it) {
            Batch bt = head;
            if (it > 0) load_batch(n0, bt);
#pragma unroll
            for (int u = 0; u < kU; ++u) {
                const bool meets = n0 + u * 64 + lane < ne && meets_tile(bt, u);
                negative = negative || (meets && !(bt.q1[u].w >= 0.0f));
                // (records that are never skipped have unbounded boxes: NaN fields or a form that is
                // not positive definite; with alpha >= 0 they can only raise a denominator)
                const float w = least_weight(bt.q0[u], bt.q1[u], txlo, txhi, tylo, tyhi);
                const bool bounded = meets && bt.q0[u].z < inf;
                sum += bounded ? w : 0.0f;
                unsigned int stored = 0u;
#pragma unroll
                for (int l = 0; l < kL; ++l) {
                    const float p = masks ? reach_p(bt.q0[u], bt.q1[u], sub[l][0], sub[l][1], sub[l][2], sub[l][3])
                                          : reach_p(bt.q0[u], bt.q1[u], txlo, txhi, tylo, tyhi);
                    const int k = weight_class(p, bt.q1[u].w);
                    // classes further than kMaxSkipClasses above the call's are never skipped (nor counted)
                    const bool classed = bounded && k >= 0 && k < kbase && kbase - k <= kMaxSkipClasses;
                    const bool live = meets && (!masks || sub_any[l]);
                    if (live && classed) atomicAdd(&hist[l][k], 1);
                    const bool gone = !live || (bounded && (p > kExactLimit || k >= kbase));
                    stored |= (gone ? 0u : (classed ? (unsigned int)(kbase - k) : 255u)) << (8 * l);
                }
                const int i = n0 + u * 64 + lane;
                if (a.store_classes && i < ne) {
                    if (masks) class_store[i] = stored;
                    else reinterpret_cast<unsigned char*>(class_store)[i] = (unsigned char)stored;
                }
            }
        }
#pragma unroll
        for (int k = 32; k > 0; k >>= 1) sum += __shfl_xor(sum, k);  // fixed order: the lists are reproducible
        const bool wneg = __ballot(negative) != 0ull;
        __syncthreads();  // red[] was read above
        if (lane == 0) {
            red[0][wave] = sum;
            red[1][wave] = wneg ? 1.0f : 0.0f;
        }
        __syncthreads();  // (also: the histograms are complete)
        float total = 0.0f, anyneg = 0.0f;
#pragma unroll
        for (int w = 0; w < kBinWaves; ++w) {
            total += w < nwaves ? red[0][w] : 0.0f;
            anyneg += w < nwaves ? red[1][w] : 0.0f;
        }
        const float floor_sum = (anyneg == 0.0f && total > 0.0f && total < inf) ? total : 0.0f;  // (an overflowed sum bounds nothing)
        if (wave < kL) {  // wave l settles list l: the first class k with (sum over classes >= k) <= budget
            constexpr int per = kBinClasses / 64;
            const float w0 = hw_exp2(-limit);
            float v[per], s = 0.0f;
            int n = 0;
#pragma unroll
            for (int j = 0; j < per; ++j) {
                const int k = lane * per + j;
                const int h = k < kbase ? hist[wave][k] : 0;
                v[j] = (float)h * hw_exp2(-(float)k * (1.0f / (float)kBinRes));
                s += v[j];
                n += h;
            }
#pragma unroll
            for (int k = 32; k > 0; k >>= 1) n += __shfl_xor(n, k);
            float after = s;  // sum over this lane's classes and those of the lanes above
#pragma unroll
            for (int dlt = 1; dlt < 64; dlt <<= 1) {
                const float o = __shfl_down(after, dlt);
                after += lane + dlt < 64 ? o : 0.0f;
            }
            float run = __shfl_down(after, 1);
            run = lane < 63 ? run : 0.0f;
            // (one percent held back for the rounding of these sums)
            const float budget = 0.99f * ((float)n * w0 + (float)a.N * fraction * floor_sum);
            int best = 0x7fffffff;
#pragma unroll
            for (int j = per - 1; j >= 0; --j) {
                run += v[j];
                best = run <= budget ? lane * per + j : best;
            }
#pragma unroll
            for (int k = 32; k > 0; k >>= 1) best = min(best, __shfl_xor(best, k));
            if (lane == 0) first_skipped_s[wave] = max(min(best, kbase), kbase - kMaxSkipClasses);
        }
        __syncthreads();
#pragma unroll
        for (int l = 0; l < kL; ++l) first_skipped[l] = first_skipped_s[l];
    }
    // code: which of the tile's four rectangles the Gaussian reaches (four lists), or 1; 0 = not listed
    auto classify = [&](int n0, const Batch& bt, int (&code)[kU], bool (&in)[kU]) {
#pragma unroll
        for (int u = 0; u < kU; ++u) {
            in[u] = n0 + u * 64 + lane < ne;
            const bool meets = in[u] && meets_tile(bt, u);
            // an unbounded box marks a record that must never be skipped; a bounded one is refined
            const bool refine = bt.q0[u].z < inf;
            int reached = 0;
            if (masks) {
#pragma unroll
                for (int w = 0; w < 4; ++w)
                    reached |= (sub_any[w] && ellipse_reaches(bt.q0[u], bt.q1[u], sub[w][0], sub[w][1], sub[w][2],
                                                              sub[w][3], first_skipped[masks ? w : 0])) ? 1 << w : 0;
            } else {
                reached = ellipse_reaches(bt.q0[u], bt.q1[u], txlo, txhi, tylo, tyhi, first_skipped[0]) ? 1 : 0;
            }
            code[u] = !meets ? 0 : (refine ? reached : (masks ? 15 : 1));
        }
    };
    // the classifying scan keeps its verdicts (one bit, or four with four lists, per candidate of this
    // lane) for the writing one when they fit in a register pair, i.e. up to 64 (16) candidates per lane
    constexpr int vbits = masks ? 4 : 1;
    const bool keep = per_wave * vbits <= 64 * 64;
    unsigned long long verdicts = 0ull;
    int cnt[kL], it = 0;
#pragma unroll
    for (int l = 0; l < kL; ++l) cnt[l] = 0;
    for (int n0 = nb; n0 < ne; n0 += 64 * kU, ++it) {
        bool in[kU];
        int code[kU];
        if (settle && a.store_classes) {  // the classes are known: a candidate is listed where its class is below the first skipped one
#pragma unroll
            for (int u = 0; u < kU; ++u) {
                const int i = n0 + u * 64 + lane;
                in[u] = i < ne;
                const unsigned int stored = !in[u] ? 0u : (masks ? class_store[i] : (unsigned int)reinterpret_cast<unsigned char*>(class_store)[i]);
                code[u] = 0;
#pragma unroll
                for (int l = 0; l < kL; ++l)
                    code[u] |= (int)((stored >> (8 * l)) & 255u) > kbase - first_skipped[l] ? 1 << l : 0;
            }
        } else {
            Batch bt = head;
            if (it > 0) load_batch(n0, bt);
            classify(n0, bt, code, in);
        }
#pragma unroll
        for (int u = 0; u < kU; ++u) {
#pragma unroll
            for (int l = 0; l < kL; ++l) cnt[l] += __popcll(__ballot((code[u] >> l) & 1));
            verdicts |= (unsigned long long)code[u] << (((it * kU + u) * vbits) & 63);
        }
    }
    if (lane == 0)
#pragma unroll
        for (int l = 0; l < kL; ++l) wsum[l][wave] = cnt[l];
    __syncthreads();
    int base[kL], total[kL];
#pragma unroll
    for (int l = 0; l < kL; ++l) {
        base[l] = total[l] = 0;
#pragma unroll
        for (int w = 0; w < kBinWaves; ++w) {
            if (w < wave) base[l] += wsum[l][w];
            total[l] += wsum[l][w];
        }
    }
    it = 0;
    for (int n0 = nb; n0 < ne; n0 += 64 * kU, ++it) {
        bool in[kU];
        int code[kU], n[kU];
        if (keep) {
#pragma unroll
            for (int u = 0; u < kU; ++u) {
                in[u] = n0 + u * 64 + lane < ne;
                code[u] = (int)((verdicts >> (((it * kU + u) * vbits) & 63)) & (unsigned long long)((1 << vbits) - 1));
                n[u] = gaussian_of(min(n0 + u * 64 + lane, M - 1));
            }
        } else {
            Batch bt = head;
            if (it > 0) load_batch(n0, bt);
            classify(n0, bt, code, in);
#pragma unroll
            for (int u = 0; u < kU; ++u) n[u] = bt.n[u];
        }
#pragma unroll
        for (int u = 0; u < kU; ++u)
#pragma unroll
            for (int l = 0; l < kL; ++l) {
                const bool listed = (code[u] >> l) & 1;
                const unsigned long long m = __ballot(listed);
                const int pos = base[l] + __popcll(m & below);
                if (listed) (masks ? a.lists + list_no(l) * a.Np : list)[pos] = n[u];
                // the slot of every candidate: its position (within the segment, at the first level,
                // where only the sign is used) or -1
                if (!masks && slot != nullptr && in[u]) slot[n[u]] = listed ? pos : -1;
                base[l] += __popcll(m);
            }
    }
    if (tid == 0)
#pragma unroll
        for (int l = 0; l < kL; ++l) a.counts[masks ? list_no(l) : list_no(0) * K + kc] = total[l];
}

template <bool kMasks>
__global__ __launch_bounds__(kMasks ? kBinThreadsMasks : kBinThreads) void k_bin(const BinArgs a) {
    bin_tile<kMasks>(a, blockIdx.x);
}

// Two sets of one-list-per-tile lists from one launch (the forward's and the backward's of a training
// step where their tilings differ): workgroups [0, first_tiles) take the tiles of `a`, the others those of
// `b`.  Both are single-level binnings over the same Gaussians (gridDim.y = 1).
__global__ __launch_bounds__(kBinThreads) void k_bin_pair(const BinArgs a, const BinArgs b, const int first_tiles) {
    const bool second = (int)blockIdx.x >= first_tiles;   // workgroup-uniform
    bin_tile<false>(second ? b : a, (int)blockIdx.x - (second ? first_tiles : 0));
}

// Exclusive prefix of the tile counts [tiles] (all images' tiles in order): offsets[i] = first record of
// tile i in the compact partial-sum array, offsets[tiles] = total number of listed entries (also stored to
// `total_out` when given: device-accessible memory of the caller).  One workgroup; fixed order.
// overflow[1] receives `stamp`, a value that names the problem the tables were built for (tables_stamp): the
// kernels that trust tables built earlier (IGS_OPT_LISTS_BUILT) compare it with their own.
__global__ __launch_bounds__(kBinThreads) void k_tile_offsets(const int* __restrict__ counts, int tiles,
                                                              long long* __restrict__ offsets, int* __restrict__ overflow,
                                                              int stamp, long long* __restrict__ total_out,
                                                              const int* __restrict__ flag, int want) {
    if (flag != nullptr && *flag != want) return;
    __shared__ long long wsum[kBinThreads / 64];
    __shared__ long long carry;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    if (tid == 0) {
        carry = 0;
        overflow[0] = 0;
        overflow[1] = stamp;
    }
    __syncthreads();
    for (int i0 = 0; i0 < tiles; i0 += kBinThreads) {
        const int i = i0 + tid;
        const long long c = i < tiles ? counts[i] : 0;
        long long incl = c;  // inclusive prefix within the wave
#pragma unroll
        for (int d = 1; d < 64; d <<= 1) {
            const long long o = __shfl_up(incl, d);
            incl += lane >= d ? o : 0;
        }
        if (lane == 63) wsum[wave] = incl;
        __syncthreads();
        long long before = carry;
        for (int w = 0; w < wave; ++w) before += wsum[w];
        if (i < tiles) offsets[i] = before + incl - c;
        __syncthreads();
        if (tid == kBinThreads - 1) carry = before + incl;
        __syncthreads();
    }
    if (tid == 0) {
        offsets[tiles] = carry;
        if (total_out != nullptr) *total_out = carry;
    }
}
