// igs_backward.h -- backward kernels: per-pixel prologue (optionally with the MSE gradient), per-Gaussian reduction on separable and general grids.
// Included by igs_gs2d.hip inside its anonymous namespace (one translation unit).
#pragma once

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
    const float4* brecs;  // separable: the backward records of the packed buffer [B][Np] (sA, skA, D'', tag)
    const long long* offsets;  // separable: first record of each tile in `partial` [B T + 1], the last = total
    long long capacity;        // separable: records that `partial` holds
    int* overflow;             // separable: [0] set where the total exceeds the capacity (nothing is stored then for the tiles that do not fit), [1] the stamp of the problem the tables were built for
    int stamp;                 // separable: tables_stamp of this call
    float* partial;  // general grids: [B][T][N][6+C]; separable: the listed entries' records, tile after tile
    float2* grid_part;  // general grids with grid gradients: [B][groups][HWp] sums of G w (t1, t2)
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
            float* rec = base + (size_t)n[g] * NF;  // one record of NF floats per column
#pragma unroll
            for (int f = 0; f < 6; ++f) rec[f] = M[g][f];
#pragma unroll
            for (int c = 0; c < C; ++c) rec[6 + c] = CG[g][c];
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
#ifndef IGS_BWD_MIN_ROWS
#define IGS_BWD_MIN_ROWS 4
#endif
constexpr int kBwdMinRows = IGS_BWD_MIN_ROWS;
#ifndef IGS_BWD_TILE_W
#define IGS_BWD_TILE_W 32
#endif
constexpr int kBwdTileW = IGS_BWD_TILE_W;

// Separable grid: lane = one Gaussian taken from the tile's list (those whose reach box meets
// the tile; the others are known to get exactly zero from it); the tile is kBwdTileW columns x
// per_tile rows.  Its pixel records stream through LDS in chunks of whole tile rows
// (double-buffered) and are read with broadcast ds_read_b128; the tile's column coordinates sit
// in LDS for the whole kernel.  A lane's sums are stored at its list position (coalesced); the
// finalize kernel finds them through the tile's slot table and takes 0 for unlisted Gaussians, so
// tiles that a Gaussian does not reach cost neither compute nor memory traffic.
//
// Exponent with the square completed along the row (write_sep_records):
//   q' = -(sA dx + skA dy)^2 + D'' dy^2 = -u^2 + cyy,   u = sA x' + (skA dy - sA px')
// with x', px' relative to the tile's middle column, so that the hoisted row term carries no more
// rounding than u itself.  Per pair: u, q' = fma(-u, u, cyy), exp2, G = <g^, c> - s (C fma), G e, and
// the sums of G e {1, u, q'} and e g^_c: 8 + 2 C instructions and one exponential.  Per row the
// sums of G e {1, u} are folded with dy into the totals of G e {1, u, dy, u dy, dy^2}, and the row's sum
// of G e u^2 is cyy times its sum of G e less its sum of G e q' (cyy is the row's constant; where it is
// large the row's weights are at most 2^-cyy, so the difference costs no accuracy that the total sees);
// at the end the moments in (u, dy) become those in (dx, dy) (dx = (u - skA dy) / sA).  Lanes whose Gaussian has no
// completed square (tag of the backward record: a form that is not positive definite, non-finite
// values) evaluate q' = (A' dx + B2' dy) dx + D' dy^2 term by term instead; what a Gaussian's sums are
// depends on the Gaussian only, not on which lanes share its wave.
#ifndef IGS_BWD_COLS_IN_REGS
#define IGS_BWD_COLS_IN_REGS 1
#endif
#ifndef IGS_BWD_TILE_SHIFT
#define IGS_BWD_TILE_SHIFT 5   // tiles per row and per image; odd, so that 8 or 16 tiles per row cycle through all columns (1 / 3 / 5 timed: c2 0.456 / 0.448 / 0.449 ms, c1 and c3 equal)
#endif
template <int C>
__global__ __launch_bounds__(kThreads, C > 8 ? 4 : 1) void k_bwd_sep(const BwdArgs a) {  // (C = 16: four waves per SIMD, i.e. at most 128 registers)
    constexpr int CP = pix_stride_sep(C), CP4 = CP / 4;
    constexpr int PX = pix_chunk(C) > kBwdTileW ? pix_chunk(C) : kBwdTileW;
    constexpr int RPC = PX / kBwdTileW;          // tile rows per chunk
    constexpr int ROW4 = kBwdTileW * CP4;        // float4 per tile row
    constexpr int E = RPC * ROW4;                // float4 per chunk
    constexpr int PRE = (E + kThreads - 1) / kThreads;
    constexpr int RS = rec_stride_of(C);
    static_assert(PX % kBwdTileW == 0 && RPC >= 1, "chunk must hold whole tile rows");
    __shared__ float4 sh[2 * E];
    __shared__ float4 xsh[kBwdTileW / 4];   // column coordinates of the tile
    __shared__ float4 xloc[kBwdTileW / 4];  // the same relative to the tile's middle column
    __shared__ float ysh[2][RPC + 1];  // row coordinates of the chunk (+1: read-ahead slot)
    IGS_GATE(a);
    // Tiles are the fastest grid dimension: consecutive workgroups (dealt round-robin to the
    // XCDs, which do not share work afterwards) then belong to different tiles, and the
    // list-position groups that have work (the low ones) are spread over all XCDs.  The tile of a
    // workgroup is shifted along its row by a few tiles per row and image: with 8 tiles per row an
    // XCD would otherwise own one tile column of every image, and the columns differ in work (at
    // the image's border the lists are shorter; a module at its initialisation puts all Gaussians
    // near the centre).  An XCD now gets one tile of every row and column of an image.
    const int b = blockIdx.z, grp = blockIdx.y;
    const int tid = threadIdx.x;
    const int ty = blockIdx.x / a.tiles_x;
    const int tx = (blockIdx.x - ty * a.tiles_x + ty * IGS_BWD_TILE_SHIFT + b * IGS_BWD_TILE_SHIFT) % a.tiles_x;
    const int t = ty * a.tiles_x + tx;
    // Tables that were not built for this problem (a caller's IGS_OPT_LISTS_BUILT on other workspaces) are
    // not read: nothing is stored, and the flag makes the finalize kernels return NaN.
    const bool foreign = a.overflow[1] != a.stamp;
    if (blockIdx.x == 0 && grp == 0 && b == 0 && tid == 0)
        a.overflow[0] = foreign || a.offsets[(size_t)gridDim.z * a.T] > a.capacity;
    if (foreign) return;  // uniform
    const int count = min(a.counts[(size_t)b * a.T + t], a.Np);
    if (grp * kThreads >= count) return;  // workgroup-uniform: no listed Gaussian left
    const long long first = a.offsets[(size_t)b * a.T + t];
    if (first + count > a.capacity) return;  // workgroup-uniform: the caller's array does not hold this tile's records
    const int* list = a.lists + ((size_t)b * a.T + t) * a.Np;
    const int pos = grp * kThreads + tid;
    const int n = pos < count ? max(list[pos], 0) : a.N;  // >= N: an unused lane (nothing is stored for it)
    const int nc = min(n, a.N - 1);
    const float* rec = a.packed + ((size_t)b * a.Np + nc) * RS;
    const float4 br = a.brecs[(size_t)b * a.Np + nc];
    const float px = rec[0], py = rec[1];
    const float rA = rec[2], rB2 = rec[3], rD = rec[4];
    float col[C];
#pragma unroll
    for (int c = 0; c < C; ++c) col[c] = a.colors[((size_t)b * a.N + nc) * C + c];
    // regular lanes: sums of G e {1, u, dy, u^2, u dy, dy^2}; the others: of G e {1, dx, dy, dx^2, dx dy, dy^2}
    float M[6], CG[C];
#pragma unroll
    for (int f = 0; f < 6; ++f) M[f] = 0.0f;
#pragma unroll
    for (int c = 0; c < C; ++c) CG[c] = 0.0f;

    const int c0 = tx * kBwdTileW;
    const int cw = min(a.Wp, c0 + kBwdTileW) - c0;  // columns of this tile, a multiple of 8
    const int r0 = ty * a.per_tile, r1 = min(a.H, r0 + a.per_tile);
    const int chunks = (r1 - r0 + RPC - 1) / RPC;
    const float4 zero = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
    const float xc = a.xs[(size_t)b * a.Wp + c0 + (cw >> 1)];
    if (tid < kBwdTileW / 4) {
        const float4 v = 4 * tid < cw ? reinterpret_cast<const float4*>(a.xs + (size_t)b * a.Wp + c0)[tid] : zero;
        xsh[tid] = v;
        xloc[tid] = 4 * tid < cw ? make_float4(v.x - xc, v.y - xc, v.z - xc, v.w - xc) : zero;
    }

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

    // Which evaluation this lane's Gaussian gets on this tile: the completed square where the record has
    // one and sA times the tile's largest |x'| stays within kSepSpanLimitBwd (NaN coordinates: term by term).
    float span = 0.0f;
    bool xbad = false;
    float xl[kBwdTileW];
#pragma unroll
    for (int i = 0; i < kBwdTileW / 4; ++i) {
        const float4 v = xloc[i];
        xl[4 * i] = v.x;
        xl[4 * i + 1] = v.y;
        xl[4 * i + 2] = v.z;
        xl[4 * i + 3] = v.w;
        span = fmaxf(span, fmaxf(fmaxf(fabsf(v.x), fabsf(v.y)), fmaxf(fabsf(v.z), fabsf(v.w))));
        xbad = xbad || !(v.x == v.x && v.y == v.y && v.z == v.z && v.w == v.w);
    }
    bool regular = br.w == 0.0f && !xbad && br.x * span <= kSepSpanLimitBwd;
    // A tile's last group of list positions is half empty on average (short lists: mostly).  A wave without
    // a listed Gaussian only helps to load the pixel records; the unused lanes of the other waves take the
    // evaluation of their wave's listed lanes, so that they do not make it run both loops.
    const bool live = pos < count;
    const bool wave_live = __ballot(live) != 0ull;
    const bool wave_regular = __ballot(live && regular) != 0ull;
    if (!live) regular = wave_regular;
    // regular lanes: sA, skA, D''; the others: A', B2', D'
    const float A = regular ? br.x : rA, B2 = regular ? br.y : rB2, D = regular ? br.z : rD;
    const float mpx = -A * (px - xc);  // regular lanes: -sA px'
    // with few channels there are registers for sA x' of the tile's columns (regular lanes)
    constexpr bool kColsInRegs = IGS_BWD_COLS_IN_REGS && C <= 4;
    float sx[kColsInRegs ? kBwdTileW : 1];
    if (kColsInRegs) {
#pragma unroll
        for (int j = 0; j < kBwdTileW; ++j) sx[j] = A * xl[j];
    }

    // the pixel record of column j of a tile row, from LDS (wave-uniform address)
    auto pixel = [&](const float4* rowrec, int j, float (&pv)[CP]) {
#pragma unroll
        for (int q4 = 0; q4 < CP4; ++q4) {
            const float4 tq = rowrec[j * CP4 + q4];
            pv[4 * q4] = tq.x;
            pv[4 * q4 + 1] = tq.y;
            pv[4 * q4 + 2] = tq.z;
            pv[4 * q4 + 3] = tq.w;
        }
    };
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
        if (!wave_live) {
            // (wave-uniform) nothing to evaluate
        } else if (regular) {
            float ynext = ycur[0];
#pragma unroll 1
            for (int rr = 0; rr < rows; ++rr) {
                // the row coordinate comes from LDS, read one row ahead: a scalar load here would
                // drain the LDS/scalar counter once per tile row
                const float yv = ynext;
                ynext = ycur[rr + 1];
                const float dy = yv - py;
                const float rowoff = fmaf(B2, dy, mpx);
                const float cyy = (D * dy) * dy;
                float R0 = 0.0f, R1 = 0.0f, RQ = 0.0f;
                const float4* rowrec = cur + rr * ROW4;
                // four pairs (columns i..i+3) from their u
                auto four_pairs = [&](int i, const float (&us)[4]) {
                    // phase 1: exponents of the 4 pairs (independent chains)
                    float qs[4], ee[4];
#pragma unroll
                    for (int j = 0; j < 4; ++j) qs[j] = fmaf(-us[j], us[j], cyy);
                    // phase 2: transcendentals back to back
#pragma unroll
                    for (int j = 0; j < 4; ++j) ee[j] = hw_exp2(qs[j]);
                    // phase 3: G = <g^, c> - s and the sums
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
                        float pv[CP];
                        pixel(rowrec, i + j, pv);
                        float Gv = pv[C];  // -s
#pragma unroll
                        for (int c = 0; c < C; ++c) Gv = fmaf(pv[c], col[c], Gv);
                        const float ge = Gv * ee[j];
                        R0 += ge;
                        R1 = fmaf(ge, us[j], R1);
                        RQ = fmaf(ge, qs[j], RQ);
#pragma unroll
                        for (int c = 0; c < C; ++c) CG[c] = fmaf(ee[j], pv[c], CG[c]);
                    }
                };
                if constexpr (kColsInRegs) {
                    // The columns' sA x' sit in registers: no coordinate reads and no loop in a row (the
                    // compiler then starts the LDS reads of a group of pixel records inside the arithmetic of
                    // the group before; reading them one group ahead by hand was no faster).  Columns beyond the
                    // tile's width (a multiple of 8, workgroup-uniform) are skipped per 8 columns.
#pragma unroll
                    for (int i = 0; i < kBwdTileW; i += 8) {
                        if (i >= cw) break;
#pragma unroll
                        for (int h = 0; h < 8; h += 4) {
                            const float us[4] = {sx[i + h] + rowoff, sx[i + h + 1] + rowoff, sx[i + h + 2] + rowoff,
                                                 sx[i + h + 3] + rowoff};
                            four_pairs(i + h, us);
                        }
                    }
                } else {
#pragma unroll 1
                    for (int i = 0; i < cw; i += 4) {
                        const float4 xq = xloc[i >> 2];
                        const float us[4] = {fmaf(A, xq.x, rowoff), fmaf(A, xq.y, rowoff), fmaf(A, xq.z, rowoff), fmaf(A, xq.w, rowoff)};
                        four_pairs(i, us);
                    }
                }
                // the tile row is complete; its sum of G e u^2 from that of G e q': u^2 = cyy - q'
                M[0] += R0;
                M[1] += R1;
                M[2] = fmaf(dy, R0, M[2]);
                M[3] += fmaf(cyy, R0, -RQ);
                M[4] = fmaf(dy, R1, M[4]);
                M[5] = fmaf(dy * dy, R0, M[5]);
            }
        } else {
            float ynext = ycur[0];
#pragma unroll 1
            for (int rr = 0; rr < rows; ++rr) {
                const float yv = ynext;
                ynext = ycur[rr + 1];
                const float dy = yv - py;
                const float cyy = (D * dy) * dy;
                const float bdy = B2 * dy;
                float R0 = 0.0f, R1 = 0.0f, R2 = 0.0f, RC[C];
#pragma unroll
                for (int c = 0; c < C; ++c) RC[c] = 0.0f;
                const float4* rowrec = cur + rr * ROW4;
#pragma unroll 1
                for (int i = 0; i < cw; i += 4) {
                    const float4 xq = xsh[i >> 2];
                    const float xs4[4] = {xq.x, xq.y, xq.z, xq.w};
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
                        const float dx = xs4[j] - px;
                        const float tt = fmaf(A, dx, bdy);
                        const float e = hw_exp2(fmaf(tt, dx, cyy));
                        float pv[CP];
                        pixel(rowrec, i + j, pv);
                        float Gv = pv[C];
#pragma unroll
                        for (int c = 0; c < C; ++c) Gv = fmaf(pv[c], col[c], Gv);
                        const float ge = Gv * e;
                        R0 += ge;
                        const float t1 = ge * dx;
                        R1 += t1;
                        R2 = fmaf(t1, dx, R2);
#pragma unroll
                        for (int c = 0; c < C; ++c) RC[c] = fmaf(e, pv[c], RC[c]);
                    }
                }
                M[0] += R0;
                M[1] += R1;
                M[3] += R2;
                M[2] = fmaf(dy, R0, M[2]);
                M[4] = fmaf(dy, R1, M[4]);
                M[5] = fmaf(dy * dy, R0, M[5]);
#pragma unroll
                for (int c = 0; c < C; ++c) CG[c] += RC[c];
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
    if (regular) {
        // moments in (u, dy) -> moments in (dx, dy), dx = (u - skA dy) / sA; in fp64: once per lane and tile
        const double iA = 1.0 / (double)A, sk = (double)B2;
        const double mu = M[1], my = M[2], muu = M[3], muy = M[4], myy = M[5];
        M[1] = (float)((mu - sk * my) * iA);
        M[3] = (float)((muu - 2.0 * sk * muy + sk * sk * myy) * (iA * iA));
        M[4] = (float)((muy - sk * myy) * iA);
    }
    if (pos < count) {
        constexpr int NF = 6 + C;
        float* out = a.partial + (size_t)(first + pos) * NF;  // one record of NF floats per list position
#pragma unroll
        for (int f = 0; f < 6; ++f) out[f] = M[f];
#pragma unroll
        for (int c = 0; c < C; ++c) out[6 + c] = CG[c];
    }
}

// General grid: the tile is a flat pixel range (multiple of 256); x and y come with the
// pixel record.  Sums are flushed into the totals once per chunk of pixel records.
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
    stream_records_lds<CP4, kPixChunk>(src, p1 - p0, sh, [&](const float4* r, const float4*) {
        float pv[CP];
#pragma unroll
        for (int q4 = 0; q4 < CP4; ++q4) {
            const float4 tq = r[q4];
            pv[4 * q4] = tq.x;
            pv[4 * q4 + 1] = tq.y;
            pv[4 * q4 + 2] = tq.z;
            pv[4 * q4 + 3] = tq.w;
        }
        // every step runs over the G Gaussians before the next one starts, so that neighbouring
        // instructions are independent (a wave issues a dependent fp32 op only every ~8 cycles, an
        // independent one every ~4.5)
        float dx[G], dy[G], ee[G], tt[G], v[G];
#pragma unroll
        for (int g = 0; g < G; ++g) dx[g] = pv[0] - px[g];
#pragma unroll
        for (int g = 0; g < G; ++g) dy[g] = pv[1] - py[g];
#pragma unroll
        for (int g = 0; g < G; ++g) tt[g] = A[g] * dx[g];
#pragma unroll
        for (int g = 0; g < G; ++g) v[g] = D[g] * dy[g];
#pragma unroll
        for (int g = 0; g < G; ++g) tt[g] = fmaf(B2[g], dy[g], tt[g]);
#pragma unroll
        for (int g = 0; g < G; ++g) v[g] = v[g] * dy[g];
#pragma unroll
        for (int g = 0; g < G; ++g) ee[g] = fmaf(tt[g], dx[g], v[g]);
#pragma unroll
        for (int g = 0; g < G; ++g) ee[g] = hw_exp2(ee[g]);
        float Gv[G], ge[G], m1[G], m2[G];
#pragma unroll
        for (int g = 0; g < G; ++g) Gv[g] = fmaf(pv[2], col[g][0], pv[2 + C]);  // <g^, c> - s
#pragma unroll
        for (int c = 1; c < C; ++c)
#pragma unroll
            for (int g = 0; g < G; ++g) Gv[g] = fmaf(pv[2 + c], col[g][c], Gv[g]);
#pragma unroll
        for (int g = 0; g < G; ++g) ge[g] = Gv[g] * ee[g];
#pragma unroll
        for (int g = 0; g < G; ++g) m1[g] = ge[g] * dx[g];
#pragma unroll
        for (int g = 0; g < G; ++g) m2[g] = ge[g] * dy[g];
#pragma unroll
        for (int g = 0; g < G; ++g) R[g][0] += ge[g];
#pragma unroll
        for (int g = 0; g < G; ++g) R[g][1] += m1[g];
#pragma unroll
        for (int g = 0; g < G; ++g) R[g][2] += m2[g];
#pragma unroll
        for (int g = 0; g < G; ++g) R[g][3] = fmaf(m1[g], dx[g], R[g][3]);
#pragma unroll
        for (int g = 0; g < G; ++g) R[g][4] = fmaf(m1[g], dy[g], R[g][4]);
#pragma unroll
        for (int g = 0; g < G; ++g) R[g][5] = fmaf(m2[g], dy[g], R[g][5]);
#pragma unroll
        for (int c = 0; c < C; ++c)
#pragma unroll
            for (int g = 0; g < G; ++g) RC[g][c] = fmaf(ee[g], pv[2 + c], RC[g][c]);
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

// ---- cross-lane sums of the fused grid gradients
// A lane of the general backward owns Gaussians, so the per-pixel sums of the grid gradients run
// across the lanes.  Instead of one 64-lane butterfly per pixel record, the records are summed in
// a transposed fashion: two records' values are merged into one register in which half of the
// lanes carry the first record's pair sums and the other half the second's, so that each level of
// the tree halves the number of live registers and a block of 64 records costs 63 merges (one per
// record) instead of 64 x 6.  Level by level the partner lane differs in bit 5, 3, 2 (within a
// group of 8 records), then 4, 0, 1 (over 8 groups): the lane whose bits are L5..L0 ends up with
// the wave's complete sum of record  (L4 + 2 L0 + 4 L1) * 8 + (L5 + 2 L3 + 4 L2)  of the block.
// The order of the additions is fixed by the lane numbers, so results are reproducible.
__device__ __forceinline__ float xl_merge32(float a, float b) {
    // v_permlane32_swap: lanes 32..63 of the first register <-> lanes 0..31 of the second
    const auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(a), __float_as_uint(b), false, false);
    return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}
__device__ __forceinline__ float xl_merge16(float a, float b) {
    // v_permlane16_swap: the odd rows (of 16 lanes) of the first <-> the even rows of the second
    const auto r = __builtin_amdgcn_permlane16_swap(__float_as_uint(a), __float_as_uint(b), false, false);
    return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}
template <int kCtrl, int kBanks>
__device__ __forceinline__ float xl_dpp(float old, float src) {  // lanes outside kBanks keep `old`
    return __uint_as_float(__builtin_amdgcn_update_dpp(__float_as_uint(old), __float_as_uint(src), kCtrl, 0xf,
                                                       kBanks, false));
}
__device__ __forceinline__ float xl_merge8(float a, float b) {
    // row_ror:8 = partner lane ^ 8; banks 0,1 (bit 3 clear) take a, banks 2,3 take b
    return xl_dpp<0x128, 0x3>(b, a) + xl_dpp<0x128, 0xc>(a, b);
}
__device__ __forceinline__ float xl_merge4(float a, float b) {
    // banks 0,2 (bit 2 clear) read lane + 4 (row_shl:4) of a, banks 1,3 read lane - 4 (row_shr:4) of b
    return xl_dpp<0x104, 0x5>(b, a) + xl_dpp<0x114, 0xa>(a, b);
}
template <int kQuadPerm>
__device__ __forceinline__ float xl_merge_quad(float a, float b, bool second) {
    const float keep = second ? b : a, send = second ? a : b;
    return keep + __uint_as_float(__builtin_amdgcn_update_dpp(0u, __float_as_uint(send), kQuadPerm, 0xf, 0xf, true));
}

// General grid with the gradients w.r.t. the grids fused in:
// d L / d x(pixel) = -sum_n G_n w_n (A dx + B dy), same with (B dx + D dy) for y.  With
// t1 = A'dx + (B2'/2) dy, t2 = (B2'/2) dx + D'dy the exponent is dx t1 + dy t2, and a lane adds
// alpha G e (t1, t2) of its G Gaussians per pixel record; the 64 lanes are summed by the
// transposed tree above, the four waves through LDS in wave order once per chunk, and the
// workgroups of the other Gaussians by k_grid_reduce, which also applies the factor -1/k of
// t1 = k (A dx + B dy).
#ifndef IGS_GRID_WAVES
#define IGS_GRID_WAVES 3
#endif
template <int C, int G>
__global__ __launch_bounds__(kThreads, C <= 8 ? IGS_GRID_WAVES : 2) void k_bwd_gen_grid(const BwdArgs a) {
    constexpr int CP = pix_stride_gen(C), CP4 = CP / 4;
    constexpr int CH = pix_chunk(C);
    constexpr int E = CH * CP4, PRE = (E + kThreads - 1) / kThreads;
    constexpr int kWaves = kThreads / 64;
    static_assert(CH % 64 == 0 && CH <= kThreads, "a chunk is whole 64-record blocks, one thread per record at the flush");
    __shared__ float4 sh[2 * E];
    __shared__ float2 wsum[2][kWaves][CH];  // per chunk parity, wave, record: the wave's grid sums
    IGS_GATE(a);
    const int b = blockIdx.z, t = blockIdx.y;
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
    int n[G];
#pragma unroll
    for (int g = 0; g < G; ++g) n[g] = (blockIdx.x * G + g) * kThreads + tid;
    float px[G], py[G], A[G], B2[G], D[G], col[G][C];
    bwd_load_gaussians<C, G>(a, b, n, px, py, A, B2, D, col);
    float hb[G], al[G];
#pragma unroll
    for (int g = 0; g < G; ++g) {
        hb[g] = 0.5f * B2[g];
        // unused lane slots (n >= N) must add nothing
        al[g] = n[g] < a.N ? a.packed[((size_t)b * a.Np + n[g]) * rec_stride_of(C) + 5] : 0.0f;
    }
    float M[G][6], CG[G][C], R[G][6], RC[G][C];
#pragma unroll
    for (int g = 0; g < G; ++g) {
#pragma unroll
        for (int f = 0; f < 6; ++f) M[g][f] = R[g][f] = 0.0f;
#pragma unroll
        for (int c = 0; c < C; ++c) CG[g][c] = RC[g][c] = 0.0f;
    }
    // the record of a 64-record block whose wave sum the tree leaves in this lane
    const int my_rec = (((lane >> 4) & 1) | ((lane & 1) << 1) | (((lane >> 1) & 1) << 2)) * 8 +
                       (((lane >> 5) & 1) | (((lane >> 3) & 1) << 1) | (((lane >> 2) & 1) << 2));
    const bool bit0 = lane & 1, bit1 = lane & 2;

    const int p0 = t * a.per_tile, p1 = min(a.HWp, p0 + a.per_tile);
    const int total = (p1 - p0) * CP4, chunks = (p1 - p0 + CH - 1) / CH;
    const float4* src = reinterpret_cast<const float4*>(a.pixrec + ((size_t)b * a.HWp + p0) * CP);
    const float4 zero = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
    float4 pre[PRE];
    auto load_records = [&](int chunk) {
#pragma unroll
        for (int i = 0; i < PRE; ++i) {
            const int e = i * kThreads + tid, ge = chunk * E + e;
            pre[i] = (e < E && ge < total) ? src[ge] : zero;   // records past the tile are zero: they add 0
        }
    };
    load_records(0);
#pragma unroll
    for (int i = 0; i < PRE; ++i) {
        const int e = i * kThreads + tid;
        if (e < E) sh[e] = pre[i];
    }
    __syncthreads();

    // One pixel record against the lane's G Gaussians; returns this lane's grid-gradient terms.
    // Every step runs over the G Gaussians before the next step starts, so that neighbouring
    // instructions are independent: a wave issues a dependent fp32 op only every ~8 cycles but an
    // independent one every ~4.5, and at three waves per SIMD that difference is not hidden.
    auto record = [&](const float4 (&r)[CP4], float& gxl, float& gyl) {
        float pv[CP];
#pragma unroll
        for (int q4 = 0; q4 < CP4; ++q4) {
            pv[4 * q4] = r[q4].x;
            pv[4 * q4 + 1] = r[q4].y;
            pv[4 * q4 + 2] = r[q4].z;
            pv[4 * q4 + 3] = r[q4].w;
        }
        float dx[G], dy[G], ee[G], t1[G], t2[G], u[G];
#pragma unroll
        for (int g = 0; g < G; ++g) dx[g] = pv[0] - px[g];
#pragma unroll
        for (int g = 0; g < G; ++g) dy[g] = pv[1] - py[g];
#pragma unroll
        for (int g = 0; g < G; ++g) t1[g] = hb[g] * dy[g];
#pragma unroll
        for (int g = 0; g < G; ++g) t2[g] = hb[g] * dx[g];
#pragma unroll
        for (int g = 0; g < G; ++g) t1[g] = fmaf(A[g], dx[g], t1[g]);
#pragma unroll
        for (int g = 0; g < G; ++g) t2[g] = fmaf(D[g], dy[g], t2[g]);
#pragma unroll
        for (int g = 0; g < G; ++g) u[g] = dy[g] * t2[g];
#pragma unroll
        for (int g = 0; g < G; ++g) ee[g] = fmaf(dx[g], t1[g], u[g]);
#pragma unroll
        for (int g = 0; g < G; ++g) ee[g] = hw_exp2(ee[g]);
        float Gv[G], ge[G], m1[G], m2[G], gw[G];
#pragma unroll
        for (int g = 0; g < G; ++g) Gv[g] = fmaf(pv[2], col[g][0], pv[2 + C]);  // <g^, c> - s
#pragma unroll
        for (int c = 1; c < C; ++c)
#pragma unroll
            for (int g = 0; g < G; ++g) Gv[g] = fmaf(pv[2 + c], col[g][c], Gv[g]);
#pragma unroll
        for (int g = 0; g < G; ++g) ge[g] = Gv[g] * ee[g];
#pragma unroll
        for (int g = 0; g < G; ++g) m1[g] = ge[g] * dx[g];
#pragma unroll
        for (int g = 0; g < G; ++g) m2[g] = ge[g] * dy[g];
#pragma unroll
        for (int g = 0; g < G; ++g) gw[g] = ge[g] * al[g];
#pragma unroll
        for (int g = 0; g < G; ++g) R[g][0] += ge[g];
#pragma unroll
        for (int g = 0; g < G; ++g) R[g][1] += m1[g];
#pragma unroll
        for (int g = 0; g < G; ++g) R[g][2] += m2[g];
#pragma unroll
        for (int g = 0; g < G; ++g) R[g][3] = fmaf(m1[g], dx[g], R[g][3]);
#pragma unroll
        for (int g = 0; g < G; ++g) R[g][4] = fmaf(m1[g], dy[g], R[g][4]);
#pragma unroll
        for (int g = 0; g < G; ++g) R[g][5] = fmaf(m2[g], dy[g], R[g][5]);
#pragma unroll
        for (int c = 0; c < C; ++c)
#pragma unroll
            for (int g = 0; g < G; ++g) RC[g][c] = fmaf(ee[g], pv[2 + c], RC[g][c]);
        // the lane's grid terms: two chains each (even / odd Gaussians), joined at the end
        float gx0 = gw[0] * t1[0], gy0 = gw[0] * t2[0];
        float gx1 = G > 1 ? gw[G > 1 ? 1 : 0] * t1[G > 1 ? 1 : 0] : 0.0f, gy1 = G > 1 ? gw[G > 1 ? 1 : 0] * t2[G > 1 ? 1 : 0] : 0.0f;
#pragma unroll
        for (int g = 2; g < G; g += 2) {
            gx0 = fmaf(gw[g], t1[g], gx0);
            gy0 = fmaf(gw[g], t2[g], gy0);
            if (g + 1 < G) {
                gx1 = fmaf(gw[g + 1], t1[g + 1], gx1);
                gy1 = fmaf(gw[g + 1], t2[g + 1], gy1);
            }
        }
        gxl = gx0 + gx1;
        gyl = gy0 + gy1;
    };

    for (int k = 0; k < chunks; ++k) {
        if (k + 1 < chunks) load_records(k + 1);
        const float4* cur = sh + (k & 1) * E;
        float x3 = 0.0f, y3 = 0.0f, x4 = 0.0f, y4 = 0.0f, x5 = 0.0f, y5 = 0.0f;  // pending partners, tree levels 3..5
#pragma unroll 1
        for (int grp = 0; grp < CH / 8; ++grp) {
            float gx[8], gy[8];
#pragma unroll
            for (int h = 0; h < 8; h += 2) {
                // the LDS reads of two records are issued together, above the work
                float4 rr[2][CP4];
#pragma unroll
                for (int u = 0; u < 2; ++u)
#pragma unroll
                    for (int i = 0; i < CP4; ++i) rr[u][i] = cur[(grp * 8 + h + u) * CP4 + i];
                __builtin_amdgcn_sched_barrier(0);
                record(rr[0], gx[h], gy[h]);
                __builtin_amdgcn_sched_barrier(0);
                record(rr[1], gx[h + 1], gy[h + 1]);
                __builtin_amdgcn_sched_barrier(0);
            }
            // The running sums are complete here: without this the compiler sinks their updates
            // below the branches that follow and keeps every record's terms alive until then.
#pragma unroll
            for (int g = 0; g < G; ++g) {
#pragma unroll
                for (int f = 0; f < 6; ++f) asm volatile("" : "+v"(R[g][f]));
#pragma unroll
                for (int c = 0; c < C; ++c) asm volatile("" : "+v"(RC[g][c]));
            }
            // levels 1-3: the 8 records of the group -> one register (lane bits 5, 3, 2)
            // (x and y alternate so that neighbouring instructions are independent)
            float ax[4], ay[4], bx[2], by[2];
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                ax[i] = xl_merge32(gx[2 * i], gx[2 * i + 1]);
                ay[i] = xl_merge32(gy[2 * i], gy[2 * i + 1]);
            }
#pragma unroll
            for (int i = 0; i < 2; ++i) {
                bx[i] = xl_merge8(ax[2 * i], ax[2 * i + 1]);
                by[i] = xl_merge8(ay[2 * i], ay[2 * i + 1]);
            }
            const float fx = xl_merge4(bx[0], bx[1]);
            const float fy = xl_merge4(by[0], by[1]);
            // levels 4-6 over the 8 groups of a block (lane bits 4, 0, 1); the branches are wave-uniform
            if (!(grp & 1)) {
                x3 = fx; y3 = fy;
            } else {
                const float wx4 = xl_merge16(x3, fx), wy4 = xl_merge16(y3, fy);
                if (!(grp & 2)) {
                    x4 = wx4; y4 = wy4;
                } else {
                    const float wx5 = xl_merge_quad<0xb1>(x4, wx4, bit0), wy5 = xl_merge_quad<0xb1>(y4, wy4, bit0);
                    if (!(grp & 4)) {
                        x5 = wx5; y5 = wy5;
                    } else {
                        const float wx6 = xl_merge_quad<0x4e>(x5, wx5, bit1), wy6 = xl_merge_quad<0x4e>(y5, wy5, bit1);
                        wsum[k & 1][wave][(grp >> 3) * 64 + my_rec] = make_float2(wx6, wy6);
                    }
                }
            }
        }
        // two-level summation of the per-Gaussian sums
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
        if (k + 1 < chunks) {
            float4* nxt = sh + ((k + 1) & 1) * E;
#pragma unroll
            for (int i = 0; i < PRE; ++i) {
                const int e = i * kThreads + tid;
                if (e < E) nxt[e] = pre[i];
            }
        }
        __syncthreads();
        // the chunk's grid sums are complete in all waves: add them in wave order.  wsum[k & 1] is
        // written again in chunk k + 2, behind the barrier that ends chunk k + 1.
        const int p = p0 + k * CH + tid;
        if (tid < CH && p < p1) {
            float2 sum = wsum[k & 1][0][tid];
#pragma unroll
            for (int w = 1; w < kWaves; ++w) {
                sum.x += wsum[k & 1][w][tid].x;
                sum.y += wsum[k & 1][w][tid].y;
            }
            a.grid_part[((size_t)b * gridDim.x + blockIdx.x) * a.HWp + p] = sum;
        }
    }
    bwd_store<C, G>(a, b, t, n, M, CG);
}
