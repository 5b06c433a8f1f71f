// igs_koleo.h -- KoLeo diversity loss: mean over rows of relu(max_{j != i} cos(x_i, x_j) + 1)
// (reference src/igs/reg.py:5-40), forward and backward, without the [B,N,N] similarity matrix
// that the reference materialises.  Included by igs_gs2d.hip inside its anonymous namespace.
//
//   k_koleo_normalize : fn = x / max(||x||, 1e-12), rows zero-padded to a multiple of 4 floats
//   k_koleo_nn        : register-tiled fn fn^T (64x64 per workgroup, 4x4 per lane, K through LDS),
//                       reduced on the fly to (max, argmax) per row and column split
//   k_koleo_combine   : splits -> nearest neighbour per row, relu(. + 1), per-workgroup sums
//   k_koleo_sum       : fixed-order sum of those -> loss
//   k_koleo_bwd       : d x_i from the neighbour of row i and from the rows whose neighbour is i
// No atomics: equal similarities resolve to the lowest column index, every sum has a fixed order.
#pragma once

constexpr int kKoleoTile = 64;        // rows and columns of a similarity tile
constexpr int kKoleoKC = 16;          // feature dimensions staged per LDS chunk
constexpr int kKoleoLd = kKoleoTile + 4;  // LDS row stride (keeps float4 reads aligned)
constexpr float kKoleoNormEps = 1e-12f;   // torch.nn.functional.normalize's default (src/igs/reg.py:22)
constexpr int kKoleoBwdRows = 4;      // rows per wave in the backward
constexpr int kKoleoBwdChunk = 256;   // feature dimensions per pass of a wave (one float4 per lane)

// Is candidate (v2, i2) to be preferred over (v1, i1)?  NaN wins and stays (torch.max propagates
// it); equal values resolve to the lower index; index -1 (no candidate) loses every tie.
__device__ __forceinline__ bool koleo_better(float v2, int i2, float v1, int i1) {
    if (v1 != v1) return false;
    if (v2 != v2) return true;
    return v2 > v1 || (v2 == v1 && (unsigned)i2 < (unsigned)i1);
}

// One wave per row: fn[row][0..Dp) and the unclamped norm.
__global__ __launch_bounds__(kThreads) void k_koleo_normalize(const float* __restrict__ x, long rows,
                                                              int D, int Dp, float* __restrict__ fn,
                                                              float* __restrict__ norm) {
    const long row = (long)blockIdx.x * (kThreads / 64) + (threadIdx.x >> 6);
    const int lane = threadIdx.x & 63;
    if (row >= rows) return;  // wave-uniform
    const float* xr = x + row * D;
    float ss = 0.0f;
    for (int d = lane; d < D; d += 64) ss = fmaf(xr[d], xr[d], ss);
#pragma unroll
    for (int k = 32; k > 0; k >>= 1) ss += __shfl_xor(ss, k);
    const float nrm = sqrtf(ss);
    const float den = fmaxf(nrm, kKoleoNormEps);
    for (int d = lane; d < Dp; d += 64) fn[row * Dp + d] = d < D ? xr[d] / den : 0.0f;
    if (lane == 0) norm[row] = nrm;
}

// Workgroup (rt, s, b): rows [64 rt, 64 rt + 64) of image b against the column tiles
// [s tiles_per_split, (s + 1) tiles_per_split).  Writes the best (value, column) per row of the
// split; the diagonal and columns >= N are excluded.
__global__ __launch_bounds__(kThreads) void k_koleo_nn(const float* __restrict__ fn, int N, int Dp,
                                                       int tiles_per_split, float* __restrict__ part_val,
                                                       int* __restrict__ part_idx) {
    __shared__ float As[kKoleoKC * kKoleoLd], Bs[kKoleoKC * kKoleoLd];
    const int b = blockIdx.z, s = blockIdx.y, S = gridDim.y;
    const int row0 = blockIdx.x * kKoleoTile;
    const int tx = threadIdx.x & 15, ty = threadIdx.x >> 4;
    const int lr = threadIdx.x >> 2, lk = (threadIdx.x & 3) * 4;  // loader: tile row, first k of a float4
    const float* img = fn + (size_t)b * N * Dp;
    const int ntiles = (N + kKoleoTile - 1) / kKoleoTile;
    const int ct0 = s * tiles_per_split, ct1 = min(ntiles, ct0 + tiles_per_split);
    const float4 zero = make_float4(0.f, 0.f, 0.f, 0.f);
    const float ninf = -__builtin_inff();
    float best[4] = {ninf, ninf, ninf, ninf};
    int bidx[4] = {-1, -1, -1, -1};
    auto stage = [&](float* dst, int first, int k0) {
        const int r = first + lr;
        const float4 v = (r < N && k0 + lk < Dp)
                             ? *reinterpret_cast<const float4*>(img + (size_t)r * Dp + k0 + lk) : zero;
        dst[(lk + 0) * kKoleoLd + lr] = v.x;
        dst[(lk + 1) * kKoleoLd + lr] = v.y;
        dst[(lk + 2) * kKoleoLd + lr] = v.z;
        dst[(lk + 3) * kKoleoLd + lr] = v.w;
    };
    const bool one_chunk = Dp <= kKoleoKC;
    if (one_chunk) stage(As, row0, 0);  // the row tile is staged once
    for (int ct = ct0; ct < ct1; ++ct) {
        const int col0 = ct * kKoleoTile;
        float acc[4][4];
#pragma unroll
        for (int r = 0; r < 4; ++r)
#pragma unroll
            for (int c = 0; c < 4; ++c) acc[r][c] = 0.0f;
        for (int k0 = 0; k0 < Dp; k0 += kKoleoKC) {
            __syncthreads();  // the previous chunk's readers are done
            if (!one_chunk) stage(As, row0, k0);
            stage(Bs, col0, k0);
            __syncthreads();
            const int kn = min(kKoleoKC, Dp - k0);
            for (int k = 0; k < kn; ++k) {
                const float4 a = *reinterpret_cast<const float4*>(&As[k * kKoleoLd + ty * 4]);
                const float4 c = *reinterpret_cast<const float4*>(&Bs[k * kKoleoLd + tx * 4]);
                const float av[4] = {a.x, a.y, a.z, a.w}, cv[4] = {c.x, c.y, c.z, c.w};
#pragma unroll
                for (int r = 0; r < 4; ++r)
#pragma unroll
                    for (int q = 0; q < 4; ++q) acc[r][q] = fmaf(av[r], cv[q], acc[r][q]);
            }
        }
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const int grow = row0 + ty * 4 + r;
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const int gcol = col0 + tx * 4 + q;
                if (gcol < N && gcol != grow && koleo_better(acc[r][q], gcol, best[r], bidx[r])) {
                    best[r] = acc[r][q];
                    bidx[r] = gcol;
                }
            }
        }
    }
    // the 16 lanes that share a row hold disjoint column sets
#pragma unroll
    for (int r = 0; r < 4; ++r) {
#pragma unroll
        for (int k = 1; k < 16; k <<= 1) {
            const float ov = __shfl_xor(best[r], k);
            const int oi = __shfl_xor(bidx[r], k);
            if (koleo_better(ov, oi, best[r], bidx[r])) {
                best[r] = ov;
                bidx[r] = oi;
            }
        }
        const int grow = row0 + ty * 4 + r;
        if (tx == 0 && grow < N) {
            part_val[((size_t)b * S + s) * N + grow] = best[r];
            part_idx[((size_t)b * S + s) * N + grow] = bidx[r];
        }
    }
}

// Thread per row: the best over the splits (in split order), the row's loss term, the gated
// neighbour index (-1: relu passes no gradient) and the workgroup's sum of terms.
__global__ __launch_bounds__(kThreads) void k_koleo_combine(const float* __restrict__ part_val,
                                                            const int* __restrict__ part_idx, int B, int N,
                                                            int S, float* __restrict__ nn_val,
                                                            int* __restrict__ nn_idx,
                                                            double* __restrict__ loss_part) {
    __shared__ double red[kThreads];
    const long row = (long)blockIdx.x * kThreads + threadIdx.x;
    double term = 0.0;
    if (row < (long)B * N) {
        const int b = (int)(row / N), n = (int)(row - (long)b * N);
        float v = -__builtin_inff();
        int idx = -1;
        for (int s = 0; s < S; ++s) {
            const float ov = part_val[((size_t)b * S + s) * N + n];
            const int oi = part_idx[((size_t)b * S + s) * N + n];
            if (koleo_better(ov, oi, v, idx)) {
                v = ov;
                idx = oi;
            }
        }
        const float t = v + 1.0f;
        nn_val[row] = v;
        nn_idx[row] = t > 0.0f ? idx : -1;
        term = t > 0.0f ? (double)t : (t != t ? (double)t : 0.0);  // relu keeps NaN
    }
    red[threadIdx.x] = term;
    __syncthreads();
    for (int k = kThreads / 2; k > 0; k >>= 1) {
        if ((int)threadIdx.x < k) red[threadIdx.x] += red[threadIdx.x + k];
        __syncthreads();
    }
    if (threadIdx.x == 0) loss_part[blockIdx.x] = red[0];
}

__global__ __launch_bounds__(kThreads) void k_koleo_sum(const double* __restrict__ loss_part, int count,
                                                        double scale, float* __restrict__ loss) {
    __shared__ double red[kThreads];
    double s = 0.0;
    for (int i = threadIdx.x; i < count; i += kThreads) s += loss_part[i];
    red[threadIdx.x] = s;
    __syncthreads();
    for (int k = kThreads / 2; k > 0; k >>= 1) {
        if ((int)threadIdx.x < k) red[threadIdx.x] += red[threadIdx.x + k];
        __syncthreads();
    }
    if (threadIdx.x == 0) *loss = (float)(red[0] * scale);
}

// A wave owns kKoleoBwdRows consecutive rows r of image b.  With j(i) the gated neighbour of row i
// and c = grad_loss / (B N):
//   d fn_r = c ( fn_j(r) + sum_{i: j(i) = r} fn_i )          (the sum in increasing i)
//   d x_r  = (d fn_r - fn_r <fn_r, d fn_r>) / ||x_r||         if ||x_r|| > 1e-12, else d fn_r / 1e-12.
// The wave scans the image's neighbour indices 64 at a time (ballot) and adds the few rows that
// point at its own; d fn is parked in the output row until <fn, d fn> is known.
__global__ __launch_bounds__(kThreads) void k_koleo_bwd(const float* __restrict__ fn,
                                                        const float* __restrict__ norm,
                                                        const int* __restrict__ nn_idx,
                                                        const float* __restrict__ grad_loss, int B, int N,
                                                        int D, int Dp, float* __restrict__ gx) {
    constexpr int RW = kKoleoBwdRows;
    const int b = blockIdx.y;
    const int lane = threadIdx.x & 63;
    const int r0 = (blockIdx.x * (kThreads / 64) + (threadIdx.x >> 6)) * RW;
    if (r0 >= N) return;  // wave-uniform
    const float c = grad_loss[0] / ((float)B * (float)N);
    const float* img = fn + (size_t)b * N * Dp;
    const int* idx = nn_idx + (size_t)b * N;
    const float4 zero = make_float4(0.f, 0.f, 0.f, 0.f);
    float dot[RW];
#pragma unroll
    for (int q = 0; q < RW; ++q) dot[q] = 0.0f;
    for (int dc = 0; dc < Dp; dc += kKoleoBwdChunk) {
        const int d = dc + 4 * lane;
        const bool live = d < Dp;
        float4 acc[RW];
#pragma unroll
        for (int q = 0; q < RW; ++q) acc[q] = zero;
        for (int i0 = 0; i0 < N; i0 += 64) {
            const int i = i0 + lane;
            const int v = i < N ? idx[i] : -1;
            unsigned long long mask = __ballot((unsigned)(v - r0) < (unsigned)RW);
            while (mask) {  // wave-uniform
                const int bit = __builtin_ctzll(mask);
                mask &= mask - 1;
                const int rr = __builtin_amdgcn_readlane(v, bit) - r0;
                const float4 f = live ? *reinterpret_cast<const float4*>(img + (size_t)(i0 + bit) * Dp + d) : zero;
#pragma unroll
                for (int q = 0; q < RW; ++q)
                    if (rr == q) {
                        acc[q].x += f.x;
                        acc[q].y += f.y;
                        acc[q].z += f.z;
                        acc[q].w += f.w;
                    }
            }
        }
#pragma unroll
        for (int q = 0; q < RW; ++q) {
            const int r = r0 + q;
            if (r >= N) break;  // wave-uniform
            const int j = idx[r];
            if (j >= 0 && live) {
                const float4 f = *reinterpret_cast<const float4*>(img + (size_t)j * Dp + d);
                acc[q].x += f.x;
                acc[q].y += f.y;
                acc[q].z += f.z;
                acc[q].w += f.w;
            }
            if (live) {
                const float4 me = *reinterpret_cast<const float4*>(img + (size_t)r * Dp + d);
                const float h[4] = {c * acc[q].x, c * acc[q].y, c * acc[q].z, c * acc[q].w};
                const float m[4] = {me.x, me.y, me.z, me.w};
                float* out = gx + ((size_t)b * N + r) * D;
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    dot[q] = fmaf(m[e], h[e], dot[q]);  // padded dimensions hold 0
                    if (d + e < D) out[d + e] = h[e];
                }
            }
        }
    }
#pragma unroll
    for (int q = 0; q < RW; ++q)
#pragma unroll
        for (int k = 32; k > 0; k >>= 1) dot[q] += __shfl_xor(dot[q], k);
    for (int dc = 0; dc < Dp; dc += kKoleoBwdChunk) {
        const int d = dc + 4 * lane;
        if (d >= Dp) continue;
#pragma unroll
        for (int q = 0; q < RW; ++q) {
            const int r = r0 + q;
            if (r >= N) break;
            const float nrm = norm[(size_t)b * N + r];
            const float4 me = *reinterpret_cast<const float4*>(img + (size_t)r * Dp + d);
            const float m[4] = {me.x, me.y, me.z, me.w};
            float* out = gx + ((size_t)b * N + r) * D;
#pragma unroll
            for (int e = 0; e < 4; ++e)
                if (d + e < D) {
                    const float h = out[d + e];  // written by this lane above
                    out[d + e] = nrm > kKoleoNormEps ? (h - m[e] * dot[q]) / nrm : h / kKoleoNormEps;
                }
        }
    }
}
