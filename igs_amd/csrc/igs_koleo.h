// igs_koleo.h -- KoLeo diversity loss: mean over rows of relu(max_{j != i} cos(x_i, x_j) + 1)
// (reference src/igs/reg.py:5-40), forward and backward, without the [B,N,N] similarity matrix
// that the reference materialises.  Included by igs_gs2d.hip inside its anonymous namespace.
//
//   k_koleo_normalize : fn = x / max(||x||, 1e-12), rows zero-padded to a multiple of 4 floats
//   k_koleo_nn_mfma   : fn fn^T on the matrix cores (fp32 MFMA), reduced on the fly to (max, argmax) per
//                       row and column split; for rows of up to 64 (padded) dimensions
//   k_koleo_nn        : the same with register-tiled vector FMAs (128x64, 64x64 or 32x32 per workgroup,
//                       K through LDS); any row length
//   k_koleo_combine   : splits -> nearest neighbour per row, relu(. + 1), per-workgroup sums
//   k_koleo_sum       : fixed-order sum of those -> loss
//   k_koleo_bwd       : d x_i from the neighbour of row i and from the rows whose neighbour is i
// No atomics: equal similarities resolve to the lowest column index, every sum has a fixed order.
#pragma once

#ifndef IGS_KOLEO_WGS_PER_CU
#define IGS_KOLEO_WGS_PER_CU 4
#endif
constexpr int kKoleoMfmaMaxD = 64;    // up to this many (padded) dimensions the similarities run on the matrix cores
constexpr int kKoleoRegK = 16;        // up to this many (padded) dimensions the row tile stays in registers
constexpr float kKoleoNormEps = 1e-12f;   // torch.nn.functional.normalize's default (src/igs/reg.py:22)
constexpr int kKoleoBwdMaxRows = 64;  // rows per wave in the backward, at most
constexpr int kKoleoBwdChunk = 2048;  // feature dimensions per pass of the backward, at most
constexpr int kKoleoBwdLds = 8192;    // floats of LDS per backward wave
constexpr int kKoleoScan = 8;         // loads of 64 neighbour indices in flight per backward wave (twice this)

// Is candidate (v2, i2) to be preferred over (v1, i1)?  NaN wins and stays (torch.max propagates
// it); equal values resolve to the lower index; index -1 (no candidate) loses every tie.
__device__ __forceinline__ bool koleo_better(float v2, int i2, float v1, int i1) {
    if (v1 != v1) return false;
    if (v2 != v2) return true;
    return v2 > v1 || (v2 == v1 && (unsigned)i2 < (unsigned)i1);
}

// One wave per row: fn[row][0..Dp) and the unclamped norm.  A row with a non-finite element
// (which makes every similarity of its image NaN in the plain expression) gets norm = NaN.
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
    bool bad = false;
    for (int d = lane; d < Dp; d += 64) {
        const float v = d < D ? xr[d] / den : 0.0f;
        bad = bad || !(fabsf(v) <= 1.0e30f);
        fn[row * Dp + d] = v;
    }
    const bool any_bad = __ballot(bad) != 0ull;
    if (lane == 0) norm[row] = any_bad ? __builtin_nanf("") : nrm;
}

// Workgroup (rt, s, b): rows [TR rt, TR rt + TR) of image b against the column tiles
// [s tiles_per_split, (s + 1) tiles_per_split) of TC columns; TR = 16 MR, TC = 16 MC: 256 lanes of
// MR x MC similarities each.  Writes the best (value, column) per row of the split; the diagonal
// and columns >= N are excluded, NaN similarities are ignored (k_koleo_combine restores them from
// the norms).  Chunks of KC feature dimensions travel global -> registers -> LDS one step ahead of
// the arithmetic (two LDS buffers, one barrier per step).  KN > 0 (= Dp <= 16): the row tile is
// read once and kept in registers, a step stages only the column tile and the k loop is unrolled
// to exactly KN; KN = 0: any Dp, 32 dimensions per step.
template <int MR, int MC, int KN>
__global__ __launch_bounds__(kThreads) void k_koleo_nn(const float* __restrict__ fn, int N, int Dp,
                                                       int tiles_per_split, float* __restrict__ part_val,
                                                       int* __restrict__ part_idx) {
    constexpr bool kRegA = KN > 0;
    constexpr int KC = kRegA ? KN : 32;
    constexpr int TR = 16 * MR, TC = 16 * MC, LDA = TR + 4, LDB = TC + 4;
    constexpr int K4 = KC / 4;                    // float4 per tile row and chunk
    constexpr int F4A = kRegA ? 0 : TR * K4;      // float4 per step: row tile (none when it is in registers),
    constexpr int F4B = TC * K4;                  // column tile
    constexpr int LPT = (F4A + F4B + kThreads - 1) / kThreads;  // loader slots per thread and step
    __shared__ float As[kRegA ? 1 : 2][KC * LDA], Bs[2][KC * LDB];
    const int b = blockIdx.z, s = blockIdx.y, S = gridDim.y;
    const int row0 = blockIdx.x * TR;
    const int tx = threadIdx.x & 15, ty = threadIdx.x >> 4;
    const float* img = fn + (size_t)b * N * Dp;
    const int ntiles = (N + TC - 1) / TC;
    const int ct0 = s * tiles_per_split, ct1 = min(ntiles, ct0 + tiles_per_split);
    const float4 zero = make_float4(0.f, 0.f, 0.f, 0.f);
    const float ninf = -__builtin_inff();
    float best[MR];
    int bidx[MR];
#pragma unroll
    for (int r = 0; r < MR; ++r) {
        best[r] = ninf;
        bidx[r] = -1;
    }
    // loader slot j of this thread: which tile (0 = rows, 1 = columns, 2 = none), tile row, first k
    auto slot = [&](int j, int& which, int& lr, int& lk) {
        const int id = j * kThreads + (int)threadIdx.x;
        which = id < F4A ? 0 : (id < F4A + F4B ? 1 : 2);
        const int e = which ? id - F4A : id;
        lr = e / K4;
        lk = (e % K4) * 4;
    };
    auto gload = [&](int j, int col0, int k0) {
        int which, lr, lk;
        slot(j, which, lr, lk);
        if (which > 1) return zero;
        const int r = (which ? col0 : row0) + lr;
        return (r < N && k0 + lk < Dp) ? *reinterpret_cast<const float4*>(img + (size_t)r * Dp + k0 + lk) : zero;
    };
    auto lstore = [&](int j, int buf, float4 v) {
        int which, lr, lk;
        slot(j, which, lr, lk);
        if (which > 1) return;
        float* dst = which ? Bs[buf] : As[kRegA ? 0 : buf];
        const int ld = which ? LDB : LDA;
        dst[(lk + 0) * ld + lr] = v.x;
        dst[(lk + 1) * ld + lr] = v.y;
        dst[(lk + 2) * ld + lr] = v.z;
        dst[(lk + 3) * ld + lr] = v.w;
    };
    float areg[kRegA ? KN : 1][MR];
    if (kRegA) {  // stage the row tile through As once
        for (int id = threadIdx.x; id < TR * K4; id += kThreads) {
            const int lr = id / K4, lk = (id % K4) * 4, r = row0 + lr;
            const float4 v = r < N ? *reinterpret_cast<const float4*>(img + (size_t)r * Dp + lk) : zero;
            As[0][(lk + 0) * LDA + lr] = v.x;
            As[0][(lk + 1) * LDA + lr] = v.y;
            As[0][(lk + 2) * LDA + lr] = v.z;
            As[0][(lk + 3) * LDA + lr] = v.w;
        }
        __syncthreads();
#pragma unroll
        for (int k = 0; k < KC; ++k)
#pragma unroll
            for (int r = 0; r < MR; ++r) areg[kRegA ? k : 0][r] = As[0][k * LDA + ty * MR + r];
    }
    const int kchunks = (Dp + KC - 1) / KC;
    const int nsteps = (ct1 - ct0) * kchunks;
    // kRegA: a step is a column tile, so a loader slot walks down the rows with a fixed stride
    const float* nptr[LPT];
    int nrow[LPT];
#pragma unroll
    for (int j = 0; j < LPT; ++j) {
        int which, lr, lk;
        slot(j, which, lr, lk);
        nrow[j] = which == 1 ? ct0 * TC + lr : N;  // N: never loads
        nptr[j] = img + (size_t)min(nrow[j], N - 1) * Dp + lk;
    }
    auto next_tile = [&](int j) {  // kRegA only: this slot's float4 of the next column tile
        const float4 v = nrow[j] < N ? *reinterpret_cast<const float4*>(nptr[j]) : zero;
        nrow[j] += TC;
        nptr[j] += (size_t)TC * Dp;
        return v;
    };
    float4 pre[LPT];
    if (nsteps > 0) {
#pragma unroll
        for (int j = 0; j < LPT; ++j) pre[j] = kRegA ? next_tile(j) : gload(j, ct0 * TC, 0);
#pragma unroll
        for (int j = 0; j < LPT; ++j) lstore(j, 0, pre[j]);
    }
    __syncthreads();
    float acc[MR][MC];
    int ct = ct0, kc = 0;
    for (int step = 0; step < nsteps; ++step) {
        const int buf = step & 1;
        const int col0 = ct * TC, k0 = kc * KC;
        int nct = ct, nkc = kc + 1;  // the step after this one
        if (nkc == kchunks) {
            nkc = 0;
            ++nct;
        }
        const bool more = step + 1 < nsteps;
        if (more) {
#pragma unroll
            for (int j = 0; j < LPT; ++j) pre[j] = kRegA ? next_tile(j) : gload(j, nct * TC, nkc * KC);
        }
        if (!kRegA && kc == 0) {
#pragma unroll
            for (int r = 0; r < MR; ++r)
#pragma unroll
                for (int q = 0; q < MC; ++q) acc[r][q] = 0.0f;
        }
        if (kRegA) {  // fully unrolled: areg stays in registers; the first product starts the sums
#pragma unroll
            for (int k = 0; k < KC; ++k) {
                float cv[MC];
#pragma unroll
                for (int q = 0; q < MC; ++q) cv[q] = Bs[buf][k * LDB + tx * MC + q];
#pragma unroll
                for (int r = 0; r < MR; ++r)
#pragma unroll
                    for (int q = 0; q < MC; ++q)
                        acc[r][q] = k == 0 ? areg[0][r] * cv[q] : fmaf(areg[kRegA ? k : 0][r], cv[q], acc[r][q]);
            }
        } else {
            const int kn = min(KC, Dp - k0);
#pragma unroll 4
            for (int k = 0; k < kn; ++k) {
                float av[MR], cv[MC];
#pragma unroll
                for (int r = 0; r < MR; ++r) av[r] = As[kRegA ? 0 : buf][k * LDA + ty * MR + r];
#pragma unroll
                for (int q = 0; q < MC; ++q) cv[q] = Bs[buf][k * LDB + tx * MC + q];
#pragma unroll
                for (int r = 0; r < MR; ++r)
#pragma unroll
                    for (int q = 0; q < MC; ++q) acc[r][q] = fmaf(av[r], cv[q], acc[r][q]);
            }
        }
        if (kc == kchunks - 1) {  // the tile's similarities are complete
            // workgroup-uniform: the last column tile, the tiles that the diagonal crosses
            if (col0 + TC > N || (col0 < row0 + TR && col0 + TC > row0)) {
#pragma unroll
                for (int r = 0; r < MR; ++r)
#pragma unroll
                    for (int q = 0; q < MC; ++q) {
                        const int gcol = col0 + tx * MC + q;
                        if (gcol >= N || gcol == row0 + ty * MR + r) acc[r][q] = ninf;
                    }
            }
#pragma unroll
            for (int r = 0; r < MR; ++r) {
                float m = acc[r][0];
#pragma unroll
                for (int q = 1; q < MC; ++q) m = fmaxf(m, acc[r][q]);
                int qi = MC - 1;
#pragma unroll
                for (int q = MC - 2; q >= 0; --q) qi = acc[r][q] == m ? q : qi;
                if (m > best[r]) {  // columns come in increasing order: the first maximum stays
                    best[r] = m;
                    bidx[r] = col0 + tx * MC + qi;
                }
            }
        }
        if (more) {
#pragma unroll
            for (int j = 0; j < LPT; ++j) lstore(j, buf ^ 1, pre[j]);
        }
        __syncthreads();
        ct = nct;
        kc = nkc;
    }
    // the 16 lanes that share a row hold disjoint column sets
#pragma unroll
    for (int r = 0; r < MR; ++r) {
#pragma unroll
        for (int k = 1; k < 16; k <<= 1) {
            const float ov = __shfl_xor(best[r], k);
            const int oi = __shfl_xor(bidx[r], k);
            if (koleo_better(ov, oi, best[r], bidx[r])) {
                best[r] = ov;
                bidx[r] = oi;
            }
        }
        const int grow = row0 + ty * MR + r;
        if (tx == 0 && grow < N) {
            part_val[((size_t)b * S + s) * N + grow] = best[r];
            part_idx[((size_t)b * S + s) * N + grow] = bidx[r];
        }
    }
}

// ---- the same search on the matrix cores, for Dp <= 64
// fp32 MFMA (v_mfma_f32_32x32x2_f32) forms the similarities; the vector ALU only keeps the running
// maximum.  A wave owns 32 query rows (the B operand, in registers for the whole kernel) and
// streams candidate rows in tiles of 32 (the A operand, from a double-buffered LDS window that the
// workgroup's four waves share): after KH = Dp/2 accumulating MFMAs lane l holds, for query
// q0 + l % 32, the similarities to the 16 candidates  c0 + 8 (r/4) + 4 (l/32) + r % 4,  r = 0..15.
// The feature index of MFMA step t is  (l/32) KH + t  for both operands (any pairing of the k
// index works as long as both agree), so a lane reads one contiguous run of KH floats per row.
// On this hardware a SIMD does not run vector instructions while its matrix core works, so every
// vector instruction per tile is paid in matrix time: the common case (a whole window of tiles
// with nothing to mask) is unrolled with immediate LDS offsets and costs 8 v_max3 and one compare
// per tile; the tiles that need masking -- the last one (candidates >= N) and the one that holds
// the wave's own queries -- take a plain loop.  Same outputs and tie rule as k_koleo_nn (lowest
// candidate index; the two half-waves of a query are merged with koleo_better at the end).
typedef float koleo_v16f __attribute__((ext_vector_type(16)));

__host__ __device__ constexpr int koleo_mfma_ld(int KH) { return ((2 * KH / 4) & 1) ? 2 * KH : 2 * KH + 4; }  // LD/4 odd
__host__ __device__ constexpr int koleo_mfma_rows(int KH) { return KH <= 6 ? 256 : (KH <= 16 ? 128 : 64); }

template <int KH>
__global__ __launch_bounds__(kThreads, 3) void k_koleo_nn_mfma(const float* __restrict__ fn, int N, int Dp,
                                                            int tiles_per_split, float* __restrict__ part_val,
                                                            int* __restrict__ part_idx) {
    constexpr int LD = koleo_mfma_ld(KH), CR = koleo_mfma_rows(KH), TPC = CR / 32;
    __shared__ __align__(16) float cs[2][CR * LD];
    const int b = blockIdx.z, s = blockIdx.y, S = gridDim.y;
    const int tid = threadIdx.x, lane = tid & 63, j = lane & 31, h = lane >> 5;
    const int q0 = blockIdx.x * 128 + __builtin_amdgcn_readfirstlane(tid >> 6) * 32;  // the wave's first query
    const int q = q0 + j;                                                              // this lane's query
    const float* img = fn + (size_t)b * N * Dp;
    const float ninf = -__builtin_inff();
    // columns of the window beyond Dp stay zero
    for (int i = tid; i < 2 * CR * LD; i += kThreads) (&cs[0][0])[i] = 0.0f;
    float bq[KH];
#pragma unroll
    for (int t = 0; t < KH; ++t) bq[t] = (q < N && h * KH + t < Dp) ? img[(size_t)q * Dp + h * KH + t] : 0.0f;
    // The query values are used here, before the loop: their loads are then known to be complete,
    // and the MFMAs inside the loop do not wait for the memory counter, which would also make them
    // wait for the prefetch of the next window issued just before them.
#pragma unroll
    for (int t = 0; t < KH; ++t) asm volatile("" : "+v"(bq[t]));
    const int ntiles = (N + 31) / 32;
    const int t0 = s * tiles_per_split, t1 = min(ntiles, t0 + tiles_per_split);
    const int row_begin = t0 * 32, row_end = min(N, t1 * 32);
    const int nchunks = (t1 - t0 + TPC - 1) / TPC;
    const int d4 = Dp / 4;                                   // float4 per row in memory
    // Staging slots of this thread: float4 number e = i kThreads + tid of a window is columns
    // 4 c4 .. 4 c4 + 3 of row r = e / d4.  The split into (r, c4) is done once, here: a division per
    // slot and window would cost more vector time than the window's MFMAs leave room for.
    constexpr int PRE = (CR * (2 * KH / 4) + kThreads - 1) / kThreads;
    float4 pre[PRE];
    int srow[PRE], scol[PRE], slds[PRE];   // row in the window (CR: no slot), first column, offset in LDS
#pragma unroll
    for (int i = 0; i < PRE; ++i) {
        const int e = i * kThreads + tid, r = e / d4, c4 = e - r * d4;
        srow[i] = e < CR * d4 ? r : CR;
        scol[i] = 4 * c4;
        slds[i] = r * LD + 4 * c4;
    }
    // (the load is unconditional, from a clamped row, and the value is selected afterwards: a load
    // behind a select of addresses would go through a flat access and a scratch copy)
    auto gload = [&](int chunk) __attribute__((always_inline)) {
        const int r0 = row_begin + chunk * CR;
#pragma unroll
        for (int i = 0; i < PRE; ++i) {
            const int r = r0 + srow[i];
            const float4 v = *reinterpret_cast<const float4*>(img + (size_t)min(r, N - 1) * Dp + scol[i]);
            const bool ok = srow[i] < CR && r < row_end;   // (component-wise: selecting whole float4 objects
            pre[i].x = ok ? v.x : 0.0f;                      //  makes the compiler select between their addresses)
            pre[i].y = ok ? v.y : 0.0f;
            pre[i].z = ok ? v.z : 0.0f;
            pre[i].w = ok ? v.w : 0.0f;
        }
    };
    auto lstore = [&](int buf) __attribute__((always_inline)) {
#pragma unroll
        for (int i = 0; i < PRE; ++i)
            if (srow[i] < CR) *reinterpret_cast<float4*>(&cs[buf][slds[i]]) = pre[i];
    };
    __syncthreads();  // the zero fill is complete
    if (nchunks > 0) {
        gload(0);
        lstore(0);
    }
    __syncthreads();
    float best = ninf;
    int bidx = -1;
    // similarities of the tile whose row for this lane starts at `row`: KH accumulating MFMAs
    auto tile_mfma = [&](const float* row) __attribute__((always_inline)) {
        float a[KH];
        if (KH % 4 == 0) {
#pragma unroll
            for (int t = 0; t < KH; t += 4) {
                const float4 v = *reinterpret_cast<const float4*>(row + t);
                a[t] = v.x; a[t + 1] = v.y; a[t + 2] = v.z; a[t + 3] = v.w;
            }
        } else {
#pragma unroll
            for (int t = 0; t < KH; t += 2) {
                const float2 v = *reinterpret_cast<const float2*>(row + t);
                a[t] = v.x; a[t + 1] = v.y;
            }
        }
        koleo_v16f acc = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int t = 0; t < KH; ++t) acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a[t], bq[t], acc, 0, 0, 0);
        return acc;
    };
    // fold a finished tile (candidates c0 .. c0 + 31) into the lane's running maximum
    auto tile_max = [&](const koleo_v16f& acc, int c0) __attribute__((always_inline)) {
        float m = acc[0];
#pragma unroll
        for (int r = 1; r < 16; ++r) m = fmaxf(m, acc[r]);
        // A lane's maximum improves ever more rarely as the scan goes on (about 1/t at tile t), so
        // the search for its position sits behind a branch that the whole wave takes together.
        if (__builtin_amdgcn_ballot_w64(m > best) != 0ull) {
            if (m > best) {  // candidates come in increasing order: the first maximum stays
                int ri = 15;
#pragma unroll
                for (int r = 14; r >= 0; --r) ri = acc[r] == m ? r : ri;
                best = m;
                bidx = c0 + 8 * (ri >> 2) + 4 * h + (ri & 3);
            }
        }
    };
    for (int k = 0; k < nchunks; ++k) {
        if (k + 1 < nchunks) gload(k + 1);
        const int c_first = row_begin + k * CR;
        const int tiles = min(TPC, t1 - t0 - k * TPC);
        const float* row0 = cs[k & 1] + j * LD + h * KH;      // this lane's row of the window's first tile
        // scalar: a whole window, all candidates < N, and the wave's own queries are not in it
        if (tiles == TPC && c_first + CR <= N && (q0 < c_first || q0 >= c_first + CR)) {
#pragma unroll
            for (int t = 0; t < TPC; t += 2) {
                const koleo_v16f a0 = tile_mfma(row0 + t * 32 * LD);
                const koleo_v16f a1 = tile_mfma(row0 + (t + 1) * 32 * LD);
                tile_max(a0, c_first + t * 32);
                tile_max(a1, c_first + (t + 1) * 32);
            }
        } else {
            for (int t = 0; t < tiles; ++t) {
                const int c0 = c_first + t * 32;
                koleo_v16f acc = tile_mfma(row0 + t * 32 * LD);
                if (c0 + 32 > N || c0 == q0) {  // scalar
#pragma unroll
                    for (int r = 0; r < 16; ++r) {
                        const int cand = c0 + 8 * (r >> 2) + 4 * h + (r & 3);
                        if (cand >= N || cand == q) acc[r] = ninf;
                    }
                }
                tile_max(acc, c0);
            }
        }
        if (k + 1 < nchunks) lstore((k + 1) & 1);
        __syncthreads();
    }
    // the two half-waves hold disjoint candidates of the same query
    const float ov = __shfl_xor(best, 32);
    const int oi = __shfl_xor(bidx, 32);
    if (koleo_better(ov, oi, best, bidx)) {
        best = ov;
        bidx = oi;
    }
    if (h == 0 && q < N) {
        part_val[((size_t)b * S + s) * N + q] = best;
        part_idx[((size_t)b * S + s) * N + q] = bidx;
    }
}

// Thread per row: the best over the splits (in split order), the row's loss term, the gated
// neighbour index (-1: relu passes no gradient) and the workgroup's sum of terms.
__global__ __launch_bounds__(kThreads) void k_koleo_combine(const float* __restrict__ part_val,
                                                            const int* __restrict__ part_idx,
                                                            const float* __restrict__ norm, int B, int N,
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
        // eight splits' loads in flight at a time (the comparisons are a short dependent chain,
        // the loads are what takes the time when few workgroups run)
        for (int s0 = 0; s0 < S; s0 += 8) {
            float ov[8];
            int oi[8];
#pragma unroll
            for (int k = 0; k < 8; ++k) {
                const int s = min(s0 + k, S - 1);
                ov[k] = part_val[((size_t)b * S + s) * N + n];
                oi[k] = part_idx[((size_t)b * S + s) * N + n];
            }
#pragma unroll
            for (int k = 0; k < 8; ++k)
                if (s0 + k < S && koleo_better(ov[k], oi[k], v, idx)) {
                    v = ov[k];
                    idx = oi[k];
                }
        }
        if (norm[row] != norm[row]) v = norm[row];  // non-finite row: NaN, which the sum below spreads
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

// One wave (a 64-thread workgroup) owns RW consecutive rows r of image b.  With j(i) the gated
// neighbour of row i and c = grad_loss / (B N):
//   d fn_r = c ( fn_j(r) + sum_{i: j(i) = r} fn_i )          (the sum in increasing i)
//   d x_r  = (d fn_r - fn_r <fn_r, d fn_r>) / ||x_r||         if ||x_r|| > 1e-12, else d fn_r / 1e-12.
// The wave scans the image's neighbour indices 512 at a time (the next 512 in flight, ballots) and
// adds the few rows that point at its own into LDS sums [RW][DC]; lane l owns the float4 groups
// l, l + 64, ... of every row, so no LDS word is shared between lanes.  More than DC
// dimensions are done DC at a time (another scan each).  d fn is parked in the output row until
// <fn_r, d fn_r> is complete.
__global__ __launch_bounds__(64) void k_koleo_bwd(const float* __restrict__ fn, const float* __restrict__ norm,
                                                  const int* __restrict__ nn_idx,
                                                  const float* __restrict__ grad_loss, int B, int N, int D,
                                                  int Dp, int RW, int DC, float* __restrict__ gx) {
    extern __shared__ __align__(16) float sums[];  // [RW][DC]
    const int b = blockIdx.y;
    const int lane = threadIdx.x;
    const int r0 = blockIdx.x * RW;
    const int rows = min(RW, N - r0);
    const float c = grad_loss[0] / ((float)B * (float)N);
    const float* img = fn + (size_t)b * N * Dp;
    const int* idx = nn_idx + (size_t)b * N;
    float* out0 = gx + ((size_t)b * N + r0) * D;
    float mydot = 0.0f;  // lane q: <fn, d fn> of row r0 + q
    float4* sums4 = reinterpret_cast<float4*>(sums);
    const int DC4 = DC / 4;
    const float4 zero = make_float4(0.f, 0.f, 0.f, 0.f);
    for (int dc = 0; dc < Dp; dc += DC) {
        const int dn4 = min(DC, Dp - dc) / 4;  // float4 per row in this pass; lane l owns l, l + 64, ...
        for (int q = 0; q < rows; ++q)
            for (int d = lane; d < dn4; d += 64) sums4[q * DC4 + d] = zero;
        // kKoleoScan x 64 neighbour indices per batch, the next batch's loads in flight meanwhile
        int v[kKoleoScan], nxt[kKoleoScan];
#pragma unroll
        for (int u = 0; u < kKoleoScan; ++u) {
            const int i = u * 64 + lane;
            nxt[u] = i < N ? idx[i] : -1;
        }
        for (int i0 = 0; i0 < N; i0 += kKoleoScan * 64) {
#pragma unroll
            for (int u = 0; u < kKoleoScan; ++u) {
                v[u] = nxt[u];
                const int i = i0 + (kKoleoScan + u) * 64 + lane;
                nxt[u] = i < N ? idx[i] : -1;
            }
#pragma unroll
            for (int u = 0; u < kKoleoScan; ++u) {
                unsigned long long mask = __ballot((unsigned)(v[u] - r0) < (unsigned)rows);
                while (mask) {  // wave-uniform
                    const int bit = __builtin_ctzll(mask);
                    mask &= mask - 1;
                    const int q = __builtin_amdgcn_readlane(v[u], bit) - r0;
                    const float4* src = reinterpret_cast<const float4*>(img + (size_t)(i0 + u * 64 + bit) * Dp + dc);
                    for (int d = lane; d < dn4; d += 64) {
                        const float4 f = src[d];
                        float4 a = sums4[q * DC4 + d];
                        a.x += f.x;
                        a.y += f.y;
                        a.z += f.z;
                        a.w += f.w;
                        sums4[q * DC4 + d] = a;
                    }
                }
            }
        }
        for (int q = 0; q < rows; ++q) {
            const int r = r0 + q;
            const int j = idx[r];
            const float4* nb = reinterpret_cast<const float4*>(img + (size_t)(j >= 0 ? j : r) * Dp + dc);
            const float4* me = reinterpret_cast<const float4*>(img + (size_t)r * Dp + dc);
            float part = 0.0f;
            for (int d = lane; d < dn4; d += 64) {
                const float4 a = sums4[q * DC4 + d];
                const float4 f = j >= 0 ? nb[d] : zero;
                const float4 m = me[d];
                const float h[4] = {c * (a.x + f.x), c * (a.y + f.y), c * (a.z + f.z), c * (a.w + f.w)};
                const float mv[4] = {m.x, m.y, m.z, m.w};
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    part = fmaf(mv[e], h[e], part);  // padded dimensions hold 0
                    if (dc + 4 * d + e < D) out0[(size_t)q * D + dc + 4 * d + e] = h[e];
                }
            }
#pragma unroll
            for (int k = 32; k > 0; k >>= 1) part += __shfl_xor(part, k);
            if (lane == q) mydot += part;
        }
    }
    for (int q = 0; q < rows; ++q) {
        const int r = r0 + q;
        const float dot = __shfl(mydot, q);
        const float nrm = norm[(size_t)b * N + r];
        const float4* me = reinterpret_cast<const float4*>(img + (size_t)r * Dp);
        for (int dc = 0; dc < Dp; dc += DC) {
            const int dn4 = min(DC, Dp - dc) / 4;
            for (int d = lane; d < dn4; d += 64) {
                const float4 m = me[dc / 4 + d];
                const float mv[4] = {m.x, m.y, m.z, m.w};
#pragma unroll
                for (int e = 0; e < 4; ++e)
                    if (dc + 4 * d + e < D) {
                        float* o = out0 + (size_t)q * D + dc + 4 * d + e;
                        const float h = *o;  // written by this lane above
                        *o = nrm > kKoleoNormEps ? (h - mv[e] * dot) / nrm : h / kKoleoNormEps;
                    }
            }
        }
    }
}
