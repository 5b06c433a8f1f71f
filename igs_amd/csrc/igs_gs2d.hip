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
//                [B,T,N,6+C] buffer which a finalize kernel sums in a fixed order (no
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

#include <atomic>
#include <mutex>
#include <type_traits>

#include "igs_hip.h"

namespace {
#include "igs_common.h"
#include "igs_pack_bin.h"
#include "igs_forward.h"
#include "igs_backward.h"
#include "igs_fit.h"
#include "igs_finalize.h"
#include "igs_grid.h"
#include "igs_koleo.h"

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
    if (N > (1 << 24)) return false;  // list-position groups of the backward are a 16-bit grid dimension
    return true;
}

#ifndef IGS_FWD_NARROW_TILES
#define IGS_FWD_NARROW_TILES 1
#endif
struct FwdGeometry {
    int wx, wcols, tiles_x, tiles_y, total_tiles;  // wx waves of wcols columns side by side
};

FwdGeometry fwd_geometry(int B, int H, int W, int C, bool sep) {
    FwdGeometry g;
    const int kFwdSepP = fwd_sep_p(C);
    if (sep) {
        // choose the wave arrangement (wx waves along the columns) that wastes the fewest lanes;
        // on a tie the squarest tile (fewest Gaussians reach it)
        long best = -1;
        g.wx = 1;
        g.wcols = 64;
        // (variants with a list per wave: the four waves' rectangles make a tile of 64 columns x 4 P rows)
        for (int wx = 1; wx <= (fwd_wave_lists(C) ? 1 : 4); wx <<= 1) {
            const long cols = (long)ceil_div(W, 64 * wx) * 64 * wx;
            const long rows = (long)ceil_div(H, kFwdSepP * (4 / wx)) * kFwdSepP * (4 / wx);
            const long area = cols * rows;
            if (best < 0 || area < best) {
                best = area;
                g.wx = wx;
            }
        }
        if (!fwd_wave_lists(C)) {
            // four waves of 32 columns x 2 P rows stacked: 32 columns x 8 P rows, the squarest tile
            const long area = (long)ceil_div(W, 32) * 32 * ceil_div(H, 8 * kFwdSepP) * 8 * kFwdSepP;
            if (IGS_FWD_NARROW_TILES && area <= best) {
                g.wx = 1;
                g.wcols = 32;
            }
        }
        g.tiles_x = ceil_div(W, g.wcols * g.wx);
        g.tiles_y = ceil_div(H, kFwdSepP * (64 / g.wcols) * (4 / g.wx));
    } else {
        g.wx = 4;
        g.wcols = 64;
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

// Two-level binning.  With many tiles and many Gaussians the cost of k_bin is every tile's
// workgroup reading all N reach boxes.  In two levels, the Gaussians are first listed per
// super-tile (kSuperX x kSuperY tiles; K workgroups per super-tile, each scanning one chunk of
// the Gaussians into its own segment of the list), then every tile scans the segments of its
// super-tile only; the finalize kernel looks at a tile's slot entry only where the super-tile
// lists the Gaussian.  The tile lists, and with them the forward, are the same as with one level;
// the finalize kernel adds the tiles in another order (super-tile by super-tile), so gradients
// agree to rounding.  Space for the super-tile lists / tables is part of the plan whenever the
// tile grid is large enough (a function of the shape only); whether a launch uses them depends
// on the work, tiles x N, or on the IGS_OPT_BIN_LEVELS_1|2 bit of the call's grid_mode argument.
struct SuperGeometry {
    int x, y, count;  // super-tiles along x, along y, per image
    int chunk, K;     // Gaussians per first-level workgroup, workgroups per super-tile
};
inline SuperGeometry super_tiles(int tiles_x, int tiles_y, int B, int N) {
    SuperGeometry g;
    g.x = ceil_div(tiles_x, kSuperX);
    g.y = ceil_div(tiles_y, kSuperY);
    g.count = g.x * g.y;
    // enough first-level workgroups for two per compute unit, of at least 4096 Gaussians each
    int K = ceil_div(512, (long)g.count * B);
    const int maxK = ceil_div(N, 4096);
    K = K > maxK ? maxK : K;
    K = K > kBinMaxChunks ? kBinMaxChunks : (K < 1 ? 1 : K);
    g.chunk = (ceil_div(N, K) + 63) & ~63;
    g.K = ceil_div(N, g.chunk);
    return g;
}
// Two binning levels from this many (Gaussian, tile) candidates per image on (measured: B=4 N=32768 on
// 240 tiles gains 4 %, B=1 N=16384 on 256 tiles nothing).
#ifndef IGS_BIN_TWO_LEVEL_FROM
#define IGS_BIN_TWO_LEVEL_FROM 6000000L
#endif
inline bool super_reserved(int tiles_x, int tiles_y) { return tiles_x * tiles_y >= 32; }
inline bool two_level(int N, int tiles_x, int tiles_y, int opts) {
    if (!super_reserved(tiles_x, tiles_y)) return false;
    if (opts & IGS_OPT_BIN_LEVELS_1) return false;
    if (opts & IGS_OPT_BIN_LEVELS_2) return true;
    return (long)N * tiles_x * tiles_y >= IGS_BIN_TWO_LEVEL_FROM;
}
// Super-tile lists of one launch: counts [B][stiles][kBinMaxChunks] then lists [B][stiles][Np].
inline size_t super_bins_bytes(int B, int stiles, int Np) {
    return ((size_t)B * stiles * kBinMaxChunks + (size_t)B * stiles * Np) * sizeof(int);
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

// The super-tile lists that follow the tile lists of a launch.
inline BinPlace super_bins_at(void* ws, size_t scratch_bytes, int B, int tiles, int Np, int stiles) {
    char* base = static_cast<char*>(ws) + align16(align16(scratch_bytes) + bins_bytes(B, tiles, Np));
    BinPlace bp;
    bp.counts = reinterpret_cast<int*>(base);
    bp.lists = bp.counts + (size_t)B * stiles * kBinMaxChunks;
    return bp;
}

// The tables of the separable backward behind the pixel records in its workspace (`scratch_bytes`:
// records + column coordinates): the tile lists (counts [B][T], lists [B][T][Np]), the super-tile lists
// where the tile grid reserves them (stiles > 0), the slot tables [B][T][Np] (Gaussian -> position in
// the tile's list, or -1) and those of the super-tiles, the tiles' first records in the compact
// partial-sum array (B T + 1 64-bit offsets, the last being the total) and a flag that the backward
// raises when that array is too small for them.
struct BwdTables {
    BinPlace bins, super;
    int* slots;
    int* super_slots;
    long long* offsets;
    int* overflow;
    size_t bytes;  // of the workspace up to the end of the tables
};
inline BwdTables bwd_tables_at(void* ws, size_t scratch_bytes, int B, int T, int Np, int stiles) {
    BwdTables t;
    char* base = static_cast<char*>(ws);
    size_t at = align16(scratch_bytes);
    t.bins = bins_at(ws, scratch_bytes, B, T);
    at += bins_bytes(B, T, Np);
    t.super = BinPlace{nullptr, nullptr};
    if (stiles > 0) {
        t.super = super_bins_at(ws, scratch_bytes, B, T, Np, stiles);
        at = align16(at) + super_bins_bytes(B, stiles, Np);
    }
    at = align16(at);
    t.slots = reinterpret_cast<int*>(base + at);
    at = align16(at + (size_t)B * T * Np * sizeof(int));
    t.super_slots = stiles > 0 ? reinterpret_cast<int*>(base + at) : nullptr;
    if (stiles > 0) at = align16(at + (size_t)B * stiles * Np * sizeof(int));
    t.offsets = reinterpret_cast<long long*>(base + at);
    at = align16(at + ((size_t)B * T + 1) * sizeof(long long));
    t.overflow = reinterpret_cast<int*>(base + at);
    t.bytes = at + 16;
    return t;
}

// A grid_mode argument of the ABI: the igs_grid_mode in the low byte, IGS_OPT_* bits above it.
inline int mode_of(int word) { return word & 0xff; }
inline int opts_of(int word) { return word & ~0xff; }

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
    if (S > IGS_FWD_MAX_SPLIT) S = IGS_FWD_MAX_SPLIT;
    if (S < 1) S = 1;
    // Gaussians per split: a multiple of 4; drop splits that would be empty
    const int nps = (ceil_div(p->n_padded, S) + 3) & ~3;
    S = ceil_div(p->n_padded, nps);
    p->fwd_split = (int)S;
    p->fwd_n_per_split = nps;
    const long groups = (long)B * ceil_div(N, kThreads * (sep ? bwd_sep_g(C) : bwd_gen_g(C))) * 4;  // waves per tile
    long T = ((long)cus * 4 * IGS_BWD_WAVES + groups - 1) / groups;     // backward: waves per SIMD wanted
    p->bwd_tiles_x = sep ? ceil_div(p->w_padded, kBwdTileW) : 1;
    p->bwd_tile_w = sep ? kBwdTileW : 0;
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
        // With as few bands as the row limit allows, whole bands of kBwdMaxRows rows and a shorter last
        // one instead of equal ones: the tiles then are the forward's wave rectangles (lists_shared).
        p->bwd_per_tile = T == ceil_div(H, kBwdMaxRows) ? (H < kBwdMaxRows ? H : kBwdMaxRows) : ceil_div(H, T);
    } else {
        p->bwd_per_tile = (ceil_div(p->hw_padded, T) + 255) & ~255;
    }
    T = (long)ceil_div(sep ? H : p->hw_padded, p->bwd_per_tile) * p->bwd_tiles_x;
    p->bwd_tiles = (int)T;
    {   // do the backward's tiles coincide with the forward's wave rectangles (tiles, with one list per tile)?
        const int frows = fwd_wave_lists(C) ? (64 / kWaveCols) * fwd_sep_p(C)
                                            : fwd_sep_p(C) * (64 / fg.wcols) * (4 / fg.wx);
        const int fcols = fwd_wave_lists(C) ? kWaveCols : fg.wcols * fg.wx;
        p->lists_shared = sep && fcols == kBwdTileW && frows == p->bwd_per_tile &&
                          ceil_div(W, fcols) == p->bwd_tiles_x;
    }
    p->fwd_tiles = sep ? fg.tiles_x * fg.tiles_y * (fwd_wave_lists(C) ? 4 : 1) : 0;
    p->pix_stride = sep ? pix_stride_sep(C) : pix_stride_gen(C);
    // records, then one bin record (8 floats) per record, then the call's skip settings (4 floats)
    // and an all-zero record, then the separable kernels' forward and backward records
    p->packed_bytes = ((uint64_t)B * p->n_padded * packed_floats_per_gaussian(C) + 4 + kZeroRecFloats) * sizeof(float);
    p->fwd_ws_bytes = S > 1 ? (uint64_t)S * B * (C + 1) * H * W * sizeof(float) : 0;
    p->pix_bytes = sep ? ((uint64_t)B * H * p->w_padded * p->pix_stride + (uint64_t)B * p->w_padded) * sizeof(float)
                       : (uint64_t)B * p->hw_padded * p->pix_stride * sizeof(float);
    const int bwd_tiles_y = sep ? (int)T / p->bwd_tiles_x : 1;
    if (sep) {  // the tile lists of each launch follow its other scratch, then the super-tile lists
        p->fwd_ws_bytes = align16(p->fwd_ws_bytes) + bins_bytes(B, p->fwd_tiles, p->n_padded);
        if (super_reserved(fg.tiles_x, fg.tiles_y))
            p->fwd_ws_bytes = align16(p->fwd_ws_bytes) +
                              super_bins_bytes(B, super_tiles(fg.tiles_x, fg.tiles_y, B, N).count, p->n_padded);
        // the backward's tables behind its pixel records: see bwd_tables_at
        p->pix_bytes = bwd_tables_at(nullptr, p->pix_bytes, B, (int)T, p->n_padded,
                                     super_reserved(p->bwd_tiles_x, bwd_tiles_y)
                                         ? super_tiles(p->bwd_tiles_x, bwd_tiles_y, B, N).count : 0).bytes;
    }
    // the partial sums when every Gaussian is listed for every tile (general grids: always); the separable
    // backward needs (listed entries) x (6 + C) floats, see igs_gs2d_forward_train
    p->partial_bytes = (uint64_t)B * T * (6 + C) * N * sizeof(float);
    return IGS_OK;
}

inline const float4* bins_of(const float* packed, int B, int Np, int RS) {
    return reinterpret_cast<const float4*>(packed + (size_t)B * Np * RS);
}
// The skip limit the pack kernel left behind the boxes.
inline const float* limit_of(const float* packed, int B, int Np, int RS) {
    return packed + (size_t)B * Np * (RS + 8);
}
// The separable kernels' records behind the zero record: the forward's [B][Np][frec_stride_of(C)], then
// the backward's [B][Np] float4.
inline const float* frecs_of(const float* packed, int B, int Np, int C) {
    return packed + (size_t)B * Np * (rec_stride_of(C) + 8) + 4 + kZeroRecFloats;
}
inline const float4* brecs_of(const float* packed, int B, int Np, int C) {
    return reinterpret_cast<const float4*>(frecs_of(packed, B, Np, C) + (size_t)B * Np * frec_stride_of(C));
}
// Skip weight of a pack call -> limit in units of the kernels' exponent (see reach_box); a weight of
// 0 (or one too small to matter) is the exact limit.
inline int limit_from_skip_weight(float skip_weight, float skip_fraction, float* limit) {
    if (!(skip_weight >= 0.0f) || skip_weight >= 1.0f) return IGS_ERR_BAD_SKIP_WEIGHT;
    if (!(skip_fraction >= 0.0f) || skip_fraction >= 1.0f) return IGS_ERR_BAD_SKIP_WEIGHT;
    *limit = skip_weight > 0.0f ? -log2f(skip_weight) : 1e30f;
    return IGS_OK;
}

// Public plan: AUTO reports the separable variant's geometry with the workspace sizes of
// whichever variant needs more.
int make_plan(int B, int N, int H, int W, int C, int grid_mode, igs_gs2d_plan_t* p) {
    grid_mode = mode_of(grid_mode);  // the option bits change no size
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

// Threads of a k_bin workgroup: four candidates per lane when there are few of them (the scans load
// and test four at a time: more threads would only be more waves to start), 1024 otherwise.
inline int bin_threads(long candidates, bool four_lists) {
    const long most = four_lists ? kBinThreadsMasks : kBinThreads;
    long t = ((candidates + 3) / 4 + 63) & ~63L;
    return (int)(t < 256 ? 256 : (t > most ? most : t));
}

// Most workgroups of a forward binning with one workgroup per wave rectangle (see igs_gs2d_forward).
#ifndef IGS_BIN_RECT_WORKGROUPS
#define IGS_BIN_RECT_WORKGROUPS 512
#endif

// LDS for the weight classes of a tile's candidates: up to 48 KB fits, with the kernel's static LDS,
// into the 64 KB that a launch gets by default; up to 128 KB (of a CU's 160) after raising the
// kernel's limit on the device, which large problems only need.
constexpr size_t kBinClassBytesDefault = 48 * 1024, kBinClassBytes = 128 * 1024;

int launch_bin(const BinArgs& a, int K, int B, hipStream_t st) {
    // (at the second level of a two-level binning the candidates are the super-tile's list: unknown here)
    const int threads = bin_threads(a.cand_lists != nullptr ? kBinThreads * 4 : (a.chunk > 0 ? a.chunk : a.N), a.sub_nx > 0);
    // LDS for the candidates' weight classes (a tile's candidates are at most all Gaussians); beyond
    // kBinClassBytes the kernel evaluates them twice instead.  Not at the first level of a two-level
    // binning, which skips by the call's skip weight alone.
    BinArgs b = a;
    const size_t class_bytes = (size_t)a.Np * (a.sub_nx > 0 ? 4 : 1);
    b.store_classes = a.chunk == 0 && class_bytes <= kBinClassBytes;
    const size_t lds = b.store_classes ? class_bytes : 0;
    if (lds > kBinClassBytesDefault) {  // once per device and kernel (the call costs tens of microseconds)
        static std::atomic<bool> raised[2][64];
        int dev = 0;
        hipError_t e = hipGetDevice(&dev);
        if (e != hipSuccess) return (int)e;
        const int which = a.sub_nx > 0 ? 1 : 0;
        if (dev < 0 || dev >= 64 || !raised[which][dev].load(std::memory_order_acquire)) {
            const void* f = which ? reinterpret_cast<const void*>(&k_bin<true>) : reinterpret_cast<const void*>(&k_bin<false>);
            e = hipFuncSetAttribute(f, hipFuncAttributeMaxDynamicSharedMemorySize, (int)kBinClassBytes);
            if (e != hipSuccess) return (int)e;
            if (dev >= 0 && dev < 64) raised[which][dev].store(true, std::memory_order_release);
        }
    }
    if (a.sub_nx > 0)
        hipLaunchKernelGGL(k_bin<true>, dim3(a.tiles_x * a.tiles_y, K, B), dim3(threads), lds, st, b);
    else
        hipLaunchKernelGGL(k_bin<false>, dim3(a.tiles_x * a.tiles_y, K, B), dim3(threads), lds, st, b);
    const hipError_t e = hipGetLastError();
    return e == hipSuccess ? IGS_OK : (int)e;
}

// Tile lists in one or two levels.  `fine` describes the tiles (its slot table, if any, included);
// `coarse` (and the super-tile slot table when `fine` has one) is used when `levels2`.
int launch_bins(BinArgs fine, int B, bool levels2, const BinPlace& coarse, int* coarse_slots, hipStream_t st) {
    fine.chunk = 0;
    fine.cand_counts = nullptr; fine.cand_lists = nullptr;
    fine.cand_K = 0; fine.cand_chunk = 0; fine.stiles_x = 0; fine.stiles = 0;
    if (!levels2) return launch_bin(fine, 1, B, st);
    const SuperGeometry sg = super_tiles(fine.tiles_x, fine.tiles_y, B, fine.N);
    BinArgs c = fine;
    c.tile_w = fine.tile_w * kSuperX; c.tile_h = fine.tile_h * kSuperY;
    c.tiles_x = sg.x; c.tiles_y = sg.y;
    c.counts = coarse.counts; c.lists = coarse.lists; c.slots = coarse_slots;
    c.chunk = sg.chunk;
    c.sub_nx = 0; c.sub_w = 0; c.sub_h = 0; c.img_lists = 0; c.row_lists = 0;  // a super-tile has one list
    int rc = launch_bin(c, sg.K, B, st);
    if (rc) return rc;
    fine.cand_counts = coarse.counts; fine.cand_lists = coarse.lists;
    fine.cand_K = sg.K; fine.cand_chunk = sg.chunk; fine.stiles_x = sg.x; fine.stiles = sg.count;
    return launch_bin(fine, 1, B, st);
}

// One launch for two single-level, one-list-per-tile binnings over the same Gaussians (k_bin_pair).
// Returns -1 (and launches nothing) where the two do not fit one launch: the class store of either beyond
// the default LDS, or four lists per tile.
int launch_bin_pair(BinArgs first, BinArgs second, int B, hipStream_t st) {
    if (first.sub_nx > 0 || second.sub_nx > 0 || first.N != second.N || first.Np != second.Np) return -1;
    const size_t class_bytes = (size_t)first.Np;
    if (class_bytes > kBinClassBytesDefault) return -1;
    for (BinArgs* a : {&first, &second}) {
        a->chunk = 0;
        a->cand_counts = nullptr; a->cand_lists = nullptr;
        a->cand_K = 0; a->cand_chunk = 0; a->stiles_x = 0; a->stiles = 0;
        a->store_classes = 1;
    }
    const int threads = bin_threads(first.N, false);
    const int n_first = first.tiles_x * first.tiles_y;
    hipLaunchKernelGGL(k_bin_pair, dim3(n_first + second.tiles_x * second.tiles_y, 1, B), dim3(threads), class_bytes, st,
                       first, second, n_first);
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
    grid_mode = mode_of(grid_mode);
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

#ifndef IGS_FWD_ONE_WAVE_FROM
#define IGS_FWD_ONE_WAVE_FROM 512
#endif
template <int C>
int launch_forward(const FwdArgs& a, bool sep, hipStream_t st) {
    const dim3 grid(((a.total_tiles + 7) / 8) * 8, a.S, 1);
    // Long list parts (c1: 1024 Gaussians per part and list) run as workgroups of one wave, four per
    // tile: c1 forward 1.10 -> 1.00 ms.  With short parts the four times as many workgroups cost
    // more than the earlier release of the wave slots gives (c3, 256 per part: +1.4 % of the step;
    // c0, 64: +3.5 %); at 512 (c2) it is even.
    if (sep && fwd_wave_lists(C) && a.Np / a.S >= IGS_FWD_ONE_WAVE_FROM)
        hipLaunchKernelGGL((k_fwd_sep<C, fwd_sep_p(C), fwd_wave_lists(C), fwd_wave_lists(C)>),
                           dim3(grid.x * 4, grid.y, 1), dim3(64), 0, st, a);
    else if (sep)
        hipLaunchKernelGGL((k_fwd_sep<C, fwd_sep_p(C), fwd_wave_lists(C)>), grid, dim3(kThreads), 0, st, a);
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

// Workgroups of the general backward along the Gaussians (= partial sums per pixel of its fused
// grid gradients).
inline int bwd_gen_groups(int N, int C) { return ceil_div(N, kThreads * bwd_gen_g(C)); }

// Separable backward: every list position up to Np is visited by a lane (one Gaussian per lane: a tile's
// last list-position group is half empty on average, which costs half as many idle lanes with groups of
// 256 as of 512 entries); workgroups past a tile's count return at once.
template <int C>
int launch_bwd_reduce(const BwdArgs& a, int B, bool sep, hipStream_t st) {
    if (sep) {
        const dim3 grid(a.T, ceil_div(a.Np, kThreads), B);
        hipLaunchKernelGGL((k_bwd_sep<C>), grid, dim3(kThreads), 0, st, a);
    } else {
        const dim3 grid(bwd_gen_groups(a.N, C), a.T, B);
        if (a.grid_part != nullptr)
            hipLaunchKernelGGL((k_bwd_gen_grid<C, bwd_gen_g(C)>), grid, dim3(kThreads), 0, st, a);
        else
            hipLaunchKernelGGL((k_bwd_gen<C, bwd_gen_g(C)>), grid, dim3(kThreads), 0, st, a);
    }
    return launch_status();
}

// Names the problem a set of backward tables belongs to (shape, tiling, binning depth): written beside the
// tables and compared by the kernels that read them.  Never 0.
inline int tables_stamp(const igs_gs2d_plan_t& plan, int opts) {
    unsigned long long h = 0x9E3779B97F4A7C15ull;
    const int tiles_y = plan.bwd_tiles / (plan.bwd_tiles_x > 0 ? plan.bwd_tiles_x : 1);
    const int v[] = {plan.B, plan.N, plan.H, plan.W, plan.C, plan.bwd_tiles, plan.bwd_tiles_x, plan.bwd_per_tile,
                     two_level(plan.N, plan.bwd_tiles_x, tiles_y, opts) ? 2 : 1};
    for (int x : v) h = (h ^ (unsigned long long)(unsigned int)x) * 0x100000001B3ull;
    const int s = (int)(h ^ (h >> 32));
    return s != 0 ? s : 1;
}

// The separable backward's tables inside its pixel workspace (plan: the separable variant's).
inline BwdTables tables_of(const igs_gs2d_plan_t& plan, void* pix_ws) {
    const int B = plan.B, T = plan.bwd_tiles, tiles_y = T / plan.bwd_tiles_x;
    const size_t scratch = ((size_t)B * plan.H * plan.w_padded * plan.pix_stride + (size_t)B * plan.w_padded) * sizeof(float);
    return bwd_tables_at(pix_ws, scratch, B, T, plan.n_padded,
                         super_reserved(plan.bwd_tiles_x, tiles_y) ? super_tiles(plan.bwd_tiles_x, tiles_y, B, plan.N).count : 0);
}

// partial_bytes: what the caller's partial-sum array holds (its capacity in records bounds what the
// separable backward may store).
int bwd_args(BwdArgs& a, const Variant& v, const float* packed, const float* colors, const float* y,
             const int64_t gs[6], int B, int N, int H, int W, int C, float* pix_ws, float* partial,
             size_t partial_bytes = 0, int opts = 0) {
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
    a.counts = nullptr; a.lists = nullptr; a.offsets = nullptr; a.overflow = nullptr;
    a.stamp = sep ? tables_stamp(plan, opts) : 0;
    a.capacity = (long long)(partial_bytes / ((6 + C) * sizeof(float)));
    a.brecs = packed ? brecs_of(packed, B, plan.n_padded, C) : nullptr;
    if (sep && pix_ws) {
        const BwdTables t = tables_of(plan, pix_ws);
        a.counts = t.bins.counts; a.lists = t.bins.lists;
        a.offsets = t.offsets; a.overflow = t.overflow;
    }
    a.partial = partial;
    a.grid_part = nullptr;
    a.flag = v.flag; a.want = v.want;
    return IGS_OK;
}

int mode_ok(int grid_mode, const int32_t* grid_flag) {
    const int opts = opts_of(grid_mode);
    if (opts & ~(IGS_OPT_NO_CULL | IGS_OPT_BIN_LEVELS_1 | IGS_OPT_BIN_LEVELS_2 | IGS_OPT_LISTS_BUILT)) return IGS_ERR_BAD_MODE;
    if ((opts & IGS_OPT_BIN_LEVELS_1) && (opts & IGS_OPT_BIN_LEVELS_2)) return IGS_ERR_BAD_MODE;
    grid_mode = mode_of(grid_mode);
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
        case IGS_ERR_BAD_SKIP_WEIGHT: return "skip weight outside [0, 1)";
        case IGS_ERR_STATIC_SCRATCH: return "problem needs more scratch than the static array holds (IGS_STATIC_SCRATCH_BYTES)";
        case IGS_ERR_STATIC_BUSY: return "the static scratch array is still in use by a call on another stream";
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

float igs_gs2d_skip_weight(int N, float eps, float tolerance) {
    if (!(tolerance > 0.0f) || !(eps > 0.0f) || N <= 0) return 0.0f;
    const double w = (double)tolerance * (double)eps / (2.0 * (double)N);
    return w < 0.5 ? (float)w : 0.5f;
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
                         int N, int C, float skip_weight, float skip_fraction, float* packed,
                         igs_stream_t stream) {
    if (!position || !cov_inv_00 || !cov_inv_01 || !cov_inv_11 || !alphas || !colors || !packed)
        return IGS_ERR_NULL_POINTER;
    if (!shape_ok(B, N, 1, 1)) return IGS_ERR_BAD_SHAPE;
    if (!channels_compiled(C)) return IGS_ERR_BAD_CHANNELS;
    float limit;
    if (const int rc = limit_from_skip_weight(skip_weight, skip_fraction, &limit)) return rc;
    const int Np = (N + 3) & ~3;
    hipLaunchKernelGGL((k_pack<false>), dim3(ceil_div(Np, kThreads), B), dim3(kThreads), 0,
                       (hipStream_t)stream, position, cov_inv_00, cov_inv_01, cov_inv_11, alphas,
                       colors, N, Np, C, rec_stride_of(C), 0.0f, limit, skip_fraction, packed,
                       const_cast<float4*>(bins_of(packed, B, Np, rec_stride_of(C))),
                       const_cast<float*>(frecs_of(packed, B, Np, C)), frec_stride_of(C),
                       const_cast<float4*>(brecs_of(packed, B, Np, C)));
    return launch_status();
}

int igs_gs2d_pack_scale_rot(const float* positions, const float* scales, const float* rotations,
                            const float* alphas, const float* colors, int B, int N, int C, float eps,
                            float skip_weight, float skip_fraction, float* packed, igs_stream_t stream) {
    if (!positions || !scales || !rotations || !alphas || !colors || !packed)
        return IGS_ERR_NULL_POINTER;
    if (!shape_ok(B, N, 1, 1)) return IGS_ERR_BAD_SHAPE;
    if (!channels_compiled(C)) return IGS_ERR_BAD_CHANNELS;
    float limit;
    if (const int rc = limit_from_skip_weight(skip_weight, skip_fraction, &limit)) return rc;
    const int Np = (N + 3) & ~3;
    hipLaunchKernelGGL((k_pack<true>), dim3(ceil_div(Np, kThreads), B), dim3(kThreads), 0,
                       (hipStream_t)stream, positions, scales, rotations, (const float*)nullptr,
                       alphas, colors, N, Np, C, rec_stride_of(C), eps, limit, skip_fraction, packed,
                       const_cast<float4*>(bins_of(packed, B, Np, rec_stride_of(C))),
                       const_cast<float*>(frecs_of(packed, B, Np, C)), frec_stride_of(C),
                       const_cast<float4*>(brecs_of(packed, B, Np, C)));
    return launch_status();
}

}  // extern "C"

namespace {
// The tile lists and slot tables of the separable backward (a = bwd_args of the separable variant, t = its
// tables); column coordinates x[b * sxb + w * sxw].
BinArgs backward_bin_args(const BwdArgs& a, const BwdTables& t, const float* x, long sxb, long sxw, const float* packed,
                          int B, int C, int opts) {
    BinArgs ba;
    ba.bins = bins_of(packed, B, a.Np, rec_stride_of(C));
    ba.limit = limit_of(packed, B, a.Np, rec_stride_of(C));
    ba.x = x; ba.y = a.y;
    ba.sxb = sxb; ba.sxw = sxw; ba.syb = a.syb; ba.syh = a.syh;
    ba.N = a.N; ba.Np = a.Np; ba.H = a.H; ba.W = a.W;
    ba.tile_w = kBwdTileW; ba.tile_h = a.per_tile;
    ba.tiles_x = a.tiles_x; ba.tiles_y = a.T / a.tiles_x;
    ba.counts = t.bins.counts; ba.lists = t.bins.lists;
    ba.slots = t.slots;
    ba.flag = a.flag; ba.want = a.want;
    ba.no_cull = (opts & IGS_OPT_NO_CULL) != 0;
    ba.sub_nx = 0; ba.sub_w = 0; ba.sub_h = 0; ba.img_lists = 0; ba.row_lists = 0;
    ba.chunk = 0;
    ba.cand_counts = nullptr; ba.cand_lists = nullptr;
    ba.cand_K = 0; ba.cand_chunk = 0; ba.stiles_x = 0; ba.stiles = 0;
    ba.store_classes = 0;
    return ba;
}

// After the backward's binning: the tiles' first records in the compact partial-sum array (and the
// total, to `total_out` as well when given: device-accessible memory, e.g. pinned host memory).
int launch_tile_offsets(const BwdArgs& a, const BwdTables& t, int B, long long* total_out, hipStream_t st) {
    hipLaunchKernelGGL(k_tile_offsets, dim3(1), dim3(kBinThreads), 0, st, (const int*)t.bins.counts, B * a.T, t.offsets,
                       t.overflow, a.stamp, total_out, a.flag, a.want);
    return launch_status();
}

int bin_backward(const BwdArgs& a, const BwdTables& t, const float* x, long sxb, long sxw, const float* packed, int B,
                 int C, int opts, long long* total_out, hipStream_t st) {
    const BinArgs ba = backward_bin_args(a, t, x, sxb, sxw, packed, B, C, opts);
    const bool levels2 = two_level(a.N, ba.tiles_x, ba.tiles_y, opts);
    const int rc = launch_bins(ba, B, levels2, t.super, levels2 ? t.super_slots : nullptr, st);
    return rc ? rc : launch_tile_offsets(a, t, B, total_out, st);
}

// pix_ws / partial: the backward's workspaces, when this is the forward of a training step: the
// backward's tile lists are then built here as well (they depend on the packed Gaussians and the grid
// only) -- one set for both passes where the tilings coincide (plan.lists_shared), else the
// backward's beside the forward's own, in one launch where that is possible; else nullptr.
int forward_impl(const float* packed, const float* x, const float* y,
                 const int64_t grid_strides[6], int grid_mode, const int32_t* grid_flag, int B,
                 int N, int H, int W, int C, float eps, float* out, float* den, void* ws,
                 size_t ws_bytes, float* pix_ws, size_t pix_bytes, long long* total_out,
                 igs_stream_t stream) {
    if (!packed || !x || !y || !grid_strides || !out || !den) return IGS_ERR_NULL_POINTER;
    int rc = mode_ok(grid_mode, grid_flag);
    if (rc) return rc;
    if (!channels_compiled(C)) return IGS_ERR_BAD_CHANNELS;
    igs_gs2d_plan_t total;
    rc = make_plan(B, N, H, W, C, grid_mode, &total);
    if (rc) return rc;
    if (total.fwd_ws_bytes > 0 && (!ws || ws_bytes < total.fwd_ws_bytes)) return IGS_ERR_WORKSPACE;
    if (((uintptr_t)packed | (uintptr_t)ws) & 15) return IGS_ERR_ALIGNMENT;  // float4 / int lists inside
    const bool train = pix_ws != nullptr;  // the backward's tile lists are built here as well
    if (train) {
        if (pix_bytes < total.pix_bytes) return IGS_ERR_WORKSPACE;
        if ((uintptr_t)pix_ws & 15) return IGS_ERR_ALIGNMENT;
    }
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
        a.frecs = frecs_of(packed, B, plan.n_padded, C);
        a.zero_rec = limit_of(packed, B, plan.n_padded, plan.rec_stride) + 4;
        a.sxb = grid_strides[0]; a.sxh = grid_strides[1]; a.sxw = grid_strides[2];
        a.syb = grid_strides[3]; a.syh = grid_strides[4]; a.syw = grid_strides[5];
        a.B = B; a.Np = plan.n_padded; a.H = H; a.W = W;
        a.S = plan.fwd_split;
        a.n_per_split = plan.fwd_n_per_split;
        a.tiles_x = fg.tiles_x; a.tiles_y = fg.tiles_y; a.total_tiles = fg.total_tiles; a.wx = fg.wx; a.wcols = fg.wcols;
        a.eps = eps; a.out = out; a.den = den; a.part = (float*)ws;
        a.counts = nullptr; a.lists = nullptr;
        a.flag = vs[i].flag; a.want = vs[i].want;
        {   // parts of unequal length only where the launch takes several rounds of resident waves (three per SIMD)
            int cus = device_cus();
            if (cus <= 0) cus = 256;
            a.ramp = 4L * fg.total_tiles * a.S > 12L * cus ? kSplitRamp : 0.0f;
        }
        // numbering of the lists: by wave rectangle (or by tile, with one list per tile), row after row
        constexpr int kHalvesL = 64 / kWaveCols;
        a.list_row = fwd_wave_lists(C) ? kHalvesL * fg.tiles_x : fg.tiles_x;
        a.list_img = fwd_wave_lists(C) ? 4 * fg.tiles_x * fg.tiles_y : fg.tiles_x * fg.tiles_y;
        const bool shared = train && plan.lists_shared;
        if (sep && shared) {
            // the backward's tiles are the forward's wave rectangles (or tiles): its lists serve both
            BwdArgs bw;
            rc = bwd_args(bw, vs[i], packed, nullptr, y, grid_strides, B, N, H, W, C, pix_ws, nullptr, 0, opts_of(grid_mode));
            if (rc) return rc;
            rc = bin_backward(bw, tables_of(plan, pix_ws), x, grid_strides[0], grid_strides[2], packed, B, C,
                              opts_of(grid_mode), total_out, st);
            if (rc) return rc;
            a.counts = bw.counts; a.lists = bw.lists;
            a.list_row = bw.tiles_x; a.list_img = bw.T;
        } else if (sep) {
            const size_t split_bytes = a.S > 1 ? (size_t)a.S * B * (C + 1) * H * W * sizeof(float) : 0;
            const BinPlace bp = bins_at(ws, split_bytes, B, plan.fwd_tiles);
            BinArgs ba;
            ba.bins = bins_of(packed, B, plan.n_padded, plan.rec_stride);
            ba.limit = limit_of(packed, B, plan.n_padded, plan.rec_stride);
            ba.x = x; ba.y = y;
            ba.sxb = a.sxb; ba.sxw = a.sxw; ba.syb = a.syb; ba.syh = a.syh;
            ba.N = N; ba.Np = plan.n_padded; ba.H = H; ba.W = W;
            ba.tile_w = fg.wcols * fg.wx; ba.tile_h = fwd_sep_p(C) * (64 / fg.wcols) * (4 / fg.wx);
            ba.tiles_x = fg.tiles_x; ba.tiles_y = fg.tiles_y;
            ba.counts = bp.counts; ba.lists = bp.lists; ba.slots = nullptr;
            ba.flag = vs[i].flag; ba.want = vs[i].want;
            ba.no_cull = (opts_of(grid_mode) & IGS_OPT_NO_CULL) != 0;
            // a list per wave of the forward: four per tile of the binning
            constexpr int kHalves = 64 / kWaveCols;
            ba.sub_nx = fwd_wave_lists(C) ? kHalves : 0;
            ba.sub_w = kWaveCols;
            ba.sub_h = kHalves * fwd_sep_p(C);
            ba.img_lists = 0; ba.row_lists = 0;
            const bool levels2 = two_level(N, fg.tiles_x, fg.tiles_y, opts_of(grid_mode));
            // Few tiles: a workgroup per wave rectangle instead of one per tile with four lists fills
            // the device better (B=1 N=16384 512x512: 28 against 72 us, measured with rectangles of
            // 64 x 16 pixels) and bounds each rectangle's denominators by itself; with many tiles the
            // four-list workgroups read the bin records a quarter as often (B=16 N=8192 256x256: 44
            // against 67 us).
            const int rect_rows = ceil_div(H, ba.sub_h), rect_cols = ceil_div(W, kWaveCols);
            if (ba.sub_nx > 0 && !levels2 && (long)B * rect_cols * rect_rows <= IGS_BIN_RECT_WORKGROUPS) {
                ba.img_lists = 4 * fg.tiles_y * fg.tiles_x;
                ba.row_lists = kHalves * fg.tiles_x;
                ba.tile_w = kWaveCols; ba.tile_h = ba.sub_h;
                ba.tiles_x = rect_cols; ba.tiles_y = rect_rows;
                ba.sub_nx = 0; ba.sub_w = 0; ba.sub_h = 0;
            }
            const BinPlace cp = levels2 ? super_bins_at(ws, split_bytes, B, plan.fwd_tiles, plan.n_padded,
                                                        super_tiles(fg.tiles_x, fg.tiles_y, B, N).count)
                                        : BinPlace{nullptr, nullptr};
            rc = -1;
            if (train) {
                // The tilings differ (small problems: the backward's tiles have fewer rows so that there
                // are enough of them): the backward's lists are built now as well, in its workspaces, in
                // the same launch where both binnings are of the plain kind, else in a second one.
                BwdArgs bw;
                rc = bwd_args(bw, vs[i], packed, nullptr, y, grid_strides, B, N, H, W, C, pix_ws, nullptr, 0, opts_of(grid_mode));
                if (rc) return rc;
                const BwdTables bt = tables_of(plan, pix_ws);
                rc = -1;
                if (!levels2 && !two_level(N, bw.tiles_x, bw.T / bw.tiles_x, opts_of(grid_mode))) {
                    rc = launch_bin_pair(ba, backward_bin_args(bw, bt, x, grid_strides[0], grid_strides[2], packed, B, C,
                                                               opts_of(grid_mode)), B, st);
                    if (rc == 0) {
                        rc = launch_tile_offsets(bw, bt, B, total_out, st);
                        if (rc) return rc;
                    }
                }
                if (rc < 0) {
                    rc = bin_backward(bw, bt, x, grid_strides[0], grid_strides[2], packed, B, C, opts_of(grid_mode),
                                      total_out, st);
                    if (rc) return rc;
                    rc = -1;
                }
            }
            if (rc < 0) rc = launch_bins(ba, B, levels2, cp, nullptr, st);
            if (rc) return rc;
            a.counts = bp.counts; a.lists = bp.lists;
        }
        IGS_DISPATCH_C(C, rc = launch_forward<kC>(a, sep, st));
        if (rc) return rc;
        if (a.S > 1) {
            hipLaunchKernelGGL(k_fwd_combine, dim3(ceil_div((long)H * W, 64), B), dim3(kThreads),
                               0, st, (const float*)ws, a.S, B, C, H * W, eps, out, den, a.flag, a.want);
            rc = launch_status();
            if (rc) return rc;
        }
    }
    return IGS_OK;
}
}  // namespace

// Scratch of igs_gs2d_forward_static_ws: one array per device, held from the load of the code
// object to the end of the process.  In host code this name is only a handle for
// hipGetSymbolAddress; the device address it yields is what the kernels get.
static __device__ __align__(256) unsigned char scratch[IGS_STATIC_SCRATCH_BYTES];

namespace {
constexpr int kMaxDevices = 64;
std::mutex g_scratch_mutex;
// Per device: the device address of `scratch` (resolved once) and the guard against overlapping use of it.
struct StaticScratch {
    void* ptr = nullptr;
    hipEvent_t done = nullptr;     // recorded behind every call outside graph capture
    hipStream_t stream = nullptr;  // of that call
    bool recorded = false;
};
StaticScratch g_scratch[kMaxDevices];

// The current device's entry (address and event made on the first call on that device).  Caller holds the mutex.
int static_scratch(StaticScratch** out) {
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return (int)e;
    if (dev < 0 || dev >= kMaxDevices) return IGS_ERR_NO_DEVICE;
    StaticScratch& s = g_scratch[dev];
    if (s.ptr == nullptr) {
        void* p = nullptr;
        e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess) return (int)e;
        if (p == nullptr) return IGS_ERR_NO_DEVICE;
        e = hipEventCreateWithFlags(&s.done, hipEventDisableTiming);
        if (e != hipSuccess) return (int)e;
        s.ptr = p;
    }
    *out = &s;
    return IGS_OK;
}
}  // namespace

extern "C" {

int igs_gs2d_forward(const float* packed, const float* x, const float* y,
                     const int64_t grid_strides[6], int grid_mode, const int32_t* grid_flag, int B,
                     int N, int H, int W, int C, float eps, float* out, float* den, void* ws,
                     size_t ws_bytes, igs_stream_t stream) {
    return forward_impl(packed, x, y, grid_strides, grid_mode, grid_flag, B, N, H, W, C, eps, out, den, ws,
                        ws_bytes, nullptr, 0, nullptr, stream);
}

int igs_gs2d_forward_train(const float* packed, const float* x, const float* y,
                           const int64_t grid_strides[6], int grid_mode, const int32_t* grid_flag,
                           int B, int N, int H, int W, int C, float eps, float* out, float* den,
                           void* ws, size_t ws_bytes, float* pix_ws, size_t pix_bytes, int64_t* listed_total,
                           igs_stream_t stream) {
    if (!pix_ws) return IGS_ERR_NULL_POINTER;
    return forward_impl(packed, x, y, grid_strides, grid_mode, grid_flag, B, N, H, W, C, eps, out, den, ws,
                        ws_bytes, pix_ws, pix_bytes, reinterpret_cast<long long*>(listed_total), stream);
}

int igs_gs2d_forward_static_ws(const float* packed, const float* x, const float* y,
                               const int64_t grid_strides[6], int grid_mode, const int32_t* grid_flag,
                               int B, int N, int H, int W, int C, float eps, float* out, float* den,
                               igs_stream_t stream) {
    int rc = mode_ok(grid_mode, grid_flag);
    if (rc) return rc;
    igs_gs2d_plan_t total;
    rc = make_plan(B, N, H, W, C, grid_mode, &total);
    if (rc) return rc;
    if (total.fwd_ws_bytes > (uint64_t)IGS_STATIC_SCRATCH_BYTES) return IGS_ERR_STATIC_SCRATCH;
    std::lock_guard<std::mutex> lock(g_scratch_mutex);  // (held over the enqueue: calls of two threads do not interleave)
    StaticScratch* sc = nullptr;
    rc = static_scratch(&sc);
    if (rc) return rc;
    hipStream_t st = (hipStream_t)stream;
    hipStreamCaptureStatus capture = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(st, &capture) != hipSuccess) capture = hipStreamCaptureStatusNone;
    const bool guarded = capture == hipStreamCaptureStatusNone;
    // the previous call's work still running on another stream: it is reading and writing the array
    if (guarded && sc->recorded && sc->stream != st && hipEventQuery(sc->done) == hipErrorNotReady)
        return IGS_ERR_STATIC_BUSY;
    rc = forward_impl(packed, x, y, grid_strides, grid_mode, grid_flag, B, N, H, W, C, eps, out, den, sc->ptr,
                      IGS_STATIC_SCRATCH_BYTES, nullptr, 0, nullptr, stream);
    if (rc == IGS_OK && guarded && hipEventRecord(sc->done, st) == hipSuccess) {
        sc->recorded = true;
        sc->stream = st;
    }
    return rc;
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

int igs_gs2d_position_penalty(const float* gs_feature, int64_t rows, int row_floats, float weight,
                              int64_t count, float* g_feature, float* loss, igs_stream_t stream) {
    if (!gs_feature || !g_feature) return IGS_ERR_NULL_POINTER;
    if (rows < 1 || rows > (int64_t)kThreads * 0x7fffffff || row_floats < 2 || count < 1) return IGS_ERR_BAD_SHAPE;
    hipLaunchKernelGGL(k_position_penalty, dim3((unsigned)((rows + kThreads - 1) / kThreads)), dim3(kThreads), 0,
                       (hipStream_t)stream, gs_feature, (long)rows, row_floats, weight, (float)(1.0 / (double)count),
                       g_feature, loss);
    return launch_status();
}

int igs_adamw_step(float* param, const float* grad, float* exp_avg, float* exp_avg_sq, int64_t count,
                   float* state, float beta1, float beta2, float eps, float weight_decay,
                   igs_stream_t stream) {
    if (!param || !grad || !exp_avg || !exp_avg_sq || !state) return IGS_ERR_NULL_POINTER;
    if (count < 1 || count > (int64_t)kThreads * 0x7fffffff) return IGS_ERR_BAD_SHAPE;
    hipStream_t st = (hipStream_t)stream;
    hipLaunchKernelGGL(k_adamw, dim3((unsigned)((count + kThreads - 1) / kThreads)), dim3(kThreads), 0, st,
                       param, grad, exp_avg, exp_avg_sq, (long)count, state, beta1, beta2, eps, weight_decay);
    return launch_status();
}

}  // extern "C"

namespace {
// What the grid gradients need beside the reduction's own arguments (all null: none wanted).
struct GridGradOut {
    const float* x = nullptr;
    const float* out = nullptr;
    const float* den = nullptr;
    const float* grad_out = nullptr;
    float eps = 0.0f;
    void* ws = nullptr;  // general variant: [B][groups][HWp] float2 partial sums
    float* g_x = nullptr;
    float* g_y = nullptr;
};

int launch_grid_standalone(const float* packed, const float* x, const float* y, const int64_t gs[6],
                           const float* out, const float* den, const float* grad_out, int B, int N, int H, int W,
                           int C, float eps, float* g_x, float* g_y, const int* flag, int want, hipStream_t st) {
    GridGradArgs a;
    a.packed = packed; a.x = x; a.y = y;
    a.sxb = gs[0]; a.sxh = gs[1]; a.sxw = gs[2];
    a.syb = gs[3]; a.syh = gs[4]; a.syw = gs[5];
    a.out = out; a.den = den; a.gout = grad_out;
    a.Np = (N + 3) & ~3; a.H = H; a.W = W;
    a.eps = eps; a.gx = g_x; a.gy = g_y;
    a.flag = flag; a.want = want;
    int rc = IGS_OK;
    IGS_DISPATCH_C(C, {
        constexpr int P = kC > 8 ? 2 : 4;
        a.tiles_per_img = ceil_div((long)H * W, kThreads * P);
        a.total_tiles = B * a.tiles_per_img;
        hipLaunchKernelGGL((k_bwd_grid<kC, P>), dim3(((a.total_tiles + 7) / 8) * 8), dim3(kThreads), 0, st, a);
        rc = launch_status();
    });
    return rc;
}

int backward_reduce(const float* packed, const float* colors, const float* y,
                    const int64_t grid_strides[6], int grid_mode, const int32_t* grid_flag,
                    int B, int N, int H, int W, int C, float* pix_ws, size_t pix_bytes,
                    float* partial, size_t partial_bytes, const GridGradOut& gg, igs_stream_t stream) {
    if (!packed || !colors || !y || !grid_strides || !pix_ws || !partial) return IGS_ERR_NULL_POINTER;
    int rc = mode_ok(grid_mode, grid_flag);
    if (rc) return rc;
    if (!channels_compiled(C)) return IGS_ERR_BAD_CHANNELS;
    igs_gs2d_plan_t total;
    rc = make_plan(B, N, H, W, C, grid_mode, &total);
    if (rc) return rc;
    if (pix_bytes < total.pix_bytes) return IGS_ERR_WORKSPACE;
    // The partial sums: general grids store every Gaussian for every tile (plan.partial_bytes); the
    // separable backward stores the listed entries only, packed tile after tile, and raises the
    // workspace's overflow flag where `partial_bytes` does not hold them (the finalize calls then
    // return NaN gradients): plan.partial_bytes always does.
    if (mode_of(grid_mode) != IGS_GRID_SEPARABLE && partial_bytes < total.partial_bytes) return IGS_ERR_WORKSPACE;
    if (partial_bytes < (size_t)(6 + C) * sizeof(float)) return IGS_ERR_WORKSPACE;
    if (((uintptr_t)packed | (uintptr_t)pix_ws) & 15) return IGS_ERR_ALIGNMENT;  // float4 / int lists inside
    hipStream_t st = (hipStream_t)stream;
    Variant vs[2];
    const int nv = variants_of(grid_mode, grid_flag, vs);
    for (int i = 0; i < nv; ++i) {
        BwdArgs a;
        rc = bwd_args(a, vs[i], packed, colors, y, grid_strides, B, N, H, W, C, pix_ws, partial, partial_bytes,
                      opts_of(grid_mode));
        if (rc) return rc;
        const bool sep = vs[i].mode == IGS_GRID_SEPARABLE;
        if (sep && !(opts_of(grid_mode) & IGS_OPT_LISTS_BUILT)) {
            // (the prologue's compact column coordinates: the same values as the grid's)
            igs_gs2d_plan_t plan;
            rc = plan_one(B, N, H, W, C, IGS_GRID_SEPARABLE, &plan);
            if (rc) return rc;
            rc = bin_backward(a, tables_of(plan, pix_ws), a.xs, a.Wp, 1, packed, B, C, opts_of(grid_mode), nullptr, st);
            if (rc) return rc;
        }
        if (gg.g_x != nullptr && !sep) a.grid_part = reinterpret_cast<float2*>(gg.ws);
        IGS_DISPATCH_C(C, rc = launch_bwd_reduce<kC>(a, B, sep, st));
        if (rc) return rc;
        if (gg.g_x == nullptr) continue;
        if (sep) {  // the pixel-major kernel of its own
            rc = launch_grid_standalone(packed, gg.x, y, grid_strides, gg.out, gg.den, gg.grad_out, B, N, H, W, C,
                                        gg.eps, gg.g_x, gg.g_y, a.flag, a.want, st);
        } else {
            hipLaunchKernelGGL(k_grid_reduce, dim3(ceil_div((long)H * W, kThreads), B), dim3(kThreads), 0, st,
                               (const float2*)gg.ws, bwd_gen_groups(N, C), H * W, a.HWp, gg.g_x, gg.g_y, a.flag,
                               a.want);
            rc = launch_status();
        }
        if (rc) return rc;
    }
    return IGS_OK;
}
}  // namespace

extern "C" {

int igs_gs2d_backward_reduce(const float* packed, const float* colors, const float* y,
                             const int64_t grid_strides[6], int grid_mode, const int32_t* grid_flag,
                             int B, int N, int H, int W, int C, float* pix_ws, size_t pix_bytes,
                             float* partial, size_t partial_bytes, igs_stream_t stream) {
    return backward_reduce(packed, colors, y, grid_strides, grid_mode, grid_flag, B, N, H, W, C, pix_ws,
                           pix_bytes, partial, partial_bytes, GridGradOut{}, stream);
}

size_t igs_gs2d_grid_workspace_bytes(int B, int N, int H, int W, int C) {
    if (!shape_ok(B, N, H, W) || !channels_compiled(C)) return 0;
    const size_t hwp = ((size_t)H * W + 3) & ~(size_t)3;
    return (size_t)B * bwd_gen_groups(N, C) * hwp * sizeof(float2);
}

int igs_gs2d_backward_with_grid(const float* packed, const float* colors, const float* x, const float* y,
                                const int64_t grid_strides[6], int grid_mode, const int32_t* grid_flag,
                                const float* out, const float* den, const float* grad_out, int B, int N,
                                int H, int W, int C, float eps, float* pix_ws, size_t pix_bytes, float* partial,
                                size_t partial_bytes, void* grid_ws, size_t grid_ws_bytes, float* g_x,
                                float* g_y, igs_stream_t stream) {
    if (!x || !out || !den || !grad_out || !g_x || !g_y) return IGS_ERR_NULL_POINTER;
    if (mode_of(grid_mode) != IGS_GRID_SEPARABLE) {  // only the general-grid kernels use grid_ws
        if (!grid_ws) return IGS_ERR_NULL_POINTER;
        if (grid_ws_bytes < igs_gs2d_grid_workspace_bytes(B, N, H, W, C)) return IGS_ERR_WORKSPACE;
        if ((uintptr_t)grid_ws & 7) return IGS_ERR_ALIGNMENT;
    }
    int rc = igs_gs2d_backward_prologue(x, y, grid_strides, grid_mode, grid_flag, out, den, grad_out, B, N,
                                        H, W, C, eps, pix_ws, pix_bytes, stream);
    if (rc) return rc;
    GridGradOut gg;
    gg.x = x; gg.out = out; gg.den = den; gg.grad_out = grad_out; gg.eps = eps;
    gg.ws = grid_ws; gg.g_x = g_x; gg.g_y = g_y;
    return backward_reduce(packed, colors, y, grid_strides, grid_mode, grid_flag, B, N, H, W, C, pix_ws,
                           pix_bytes, partial, partial_bytes, gg, stream);
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
    return launch_grid_standalone(packed, x, y, grid_strides, out, den, grad_out, B, N, H, W, C, eps, g_x, g_y,
                                  nullptr, 0, (hipStream_t)stream);
}

// Launches a finalize kernel in the layout that suits the problem size: 8 t-lanes x 32 Gaussians
// per workgroup, or 32 x 8 when that would give fewer than two workgroups per compute unit.
#define IGS_FINALIZE_LAUNCH(B, N, KERNEL, ...)                                                      \
    do {                                                                                            \
        if ((long)(B) * ceil_div((N), 256 / kFinWide) >= 512) {                                     \
            constexpr int kFT = kFinWide;                                                           \
            hipLaunchKernelGGL(KERNEL, dim3(ceil_div((N), 256 / kFT), (B)), dim3(kThreads), 0,      \
                               __VA_ARGS__);                                                        \
        } else {                                                                                    \
            constexpr int kFT = kFinDeep;                                                           \
            hipLaunchKernelGGL(KERNEL, dim3(ceil_div((N), 256 / kFT), (B)), dim3(kThreads), 0,      \
                               __VA_ARGS__);                                                        \
        }                                                                                           \
    } while (0)

// Which finalize kernel: a group of lanes per Gaussian (k_bwd_finalize_listed) after a two-level
// binning and wherever the Gaussians alone fill the device; else t-lanes x Gaussians
// (k_bwd_finalize*), which also spreads the tiles of a Gaussian over lanes.
#ifndef IGS_FIN_GROUPS_FROM
#define IGS_FIN_GROUPS_FROM 65536L
#endif
#ifndef IGS_FIN_GROUPS_MAX_TILES
#define IGS_FIN_GROUPS_MAX_TILES 128
#endif
static bool finalize_by_groups(const SuperSlots& sup, int B, int N, int T) {
    if (sup.cslots != nullptr) return true;
    return (long)B * N >= IGS_FIN_GROUPS_FROM && T <= IGS_FIN_GROUPS_MAX_TILES;
}

// What the finalize kernels need of the backward that ran: T of the separable (or only) variant and of
// the general variant under AUTO; the separable backward's tables in its pixel workspace (slot tables,
// the tiles' first records in the compact partial array, the overflow flag; none on general grids) and
// the super-tile slot tables when it binned in two levels.
struct FinalizeTables {
    int T, T_alt;
    const int* slots;
    const long long* offsets;
    const int* overflow;
    int stamp;
    SuperSlots sup;
};
static int finalize_tables(int grid_mode, int B, int N, int H, int W, int C, const float* pix_ws, FinalizeTables* ft) {
    const int opts = opts_of(grid_mode);
    grid_mode = mode_of(grid_mode);
    igs_gs2d_plan_t plan;
    int rc = plan_one(B, N, H, W, C, grid_mode == IGS_GRID_AUTO ? IGS_GRID_SEPARABLE : grid_mode, &plan);
    if (rc) return rc;
    ft->T = plan.bwd_tiles;
    ft->T_alt = plan.bwd_tiles;
    ft->slots = nullptr; ft->offsets = nullptr; ft->overflow = nullptr;
    ft->stamp = 0;
    ft->sup = SuperSlots{nullptr, 1, 1, 1, 1};
    if (grid_mode != IGS_GRID_GENERAL) {
        if (!pix_ws) return IGS_ERR_NULL_POINTER;
        const BwdTables t = tables_of(plan, const_cast<float*>(pix_ws));
        ft->slots = t.slots; ft->offsets = t.offsets; ft->overflow = t.overflow;
        ft->stamp = tables_stamp(plan, opts);
        const int tiles_y = plan.bwd_tiles / plan.bwd_tiles_x;
        if (two_level(N, plan.bwd_tiles_x, tiles_y, opts)) {
            const SuperGeometry sg = super_tiles(plan.bwd_tiles_x, tiles_y, B, N);
            ft->sup.cslots = t.super_slots;
            ft->sup.tiles_x = plan.bwd_tiles_x;
            ft->sup.tiles_y = tiles_y;
            ft->sup.stiles_x = sg.x;
            ft->sup.stiles = sg.count;
        }
    }
    if (grid_mode == IGS_GRID_AUTO) {
        rc = plan_one(B, N, H, W, C, IGS_GRID_GENERAL, &plan);
        if (rc) return rc;
        ft->T_alt = plan.bwd_tiles;
    }
    return IGS_OK;
}

int igs_gs2d_finalize_covinv(const float* partial, const float* pix_ws, int grid_mode, const int32_t* grid_flag,
                             const float* cov_inv_00, const float* cov_inv_01,
                             const float* cov_inv_11, const float* alphas, int B, int N, int H, int W,
                             int C, float* g_position, float* g_cov_inv_00, float* g_cov_inv_01,
                             float* g_cov_inv_11, float* g_alphas, float* g_colors,
                             igs_stream_t stream) {
    if (!partial || !cov_inv_00 || !cov_inv_01 || !cov_inv_11 || !alphas) return IGS_ERR_NULL_POINTER;
    int rc = mode_ok(grid_mode, grid_flag);
    if (rc) return rc;
    FinalizeTables ft;
    rc = finalize_tables(grid_mode, B, N, H, W, C, pix_ws, &ft);
    if (rc) return rc;
    const int32_t* flag = mode_of(grid_mode) == IGS_GRID_AUTO ? grid_flag : nullptr;
    if (finalize_by_groups(ft.sup, B, N, ft.T))
        launch_finalize_listed<0>(FinalizeArgs{partial, ft.T, ft.T_alt, flag, ft.slots, ft.offsets, ft.overflow, ft.stamp, ft.sup,
                                               (N + 3) & ~3, N, C, C, cov_inv_00,
                                               cov_inv_01, cov_inv_11, alphas, 0.0f, g_position, g_cov_inv_00,
                                               g_cov_inv_01, g_cov_inv_11, g_alphas, g_colors},
                                  B, (hipStream_t)stream);
    else
        IGS_FINALIZE_LAUNCH(B, N, (k_bwd_finalize<false, kFT>),
                           (hipStream_t)stream, partial, ft.T, flag, ft.T_alt, ft.slots, ft.offsets, ft.overflow, ft.stamp,
                           (N + 3) & ~3, cov_inv_00,
                           cov_inv_01, cov_inv_11, alphas, N, C, 0.0f, g_position,
                           g_cov_inv_00, g_cov_inv_01, g_cov_inv_11, g_alphas, g_colors);
    return launch_status();
}

int igs_gs2d_finalize_scale_rot(const float* partial, const float* pix_ws, int grid_mode, const int32_t* grid_flag,
                                const float* scales, const float* rotations, const float* alphas,
                                int B, int N, int H, int W, int C, float eps, float* g_positions,
                                float* g_scales, float* g_rotations, float* g_alphas, float* g_colors,
                                igs_stream_t stream) {
    if (!partial || !scales || !rotations || !alphas) return IGS_ERR_NULL_POINTER;
    int rc = mode_ok(grid_mode, grid_flag);
    if (rc) return rc;
    FinalizeTables ft;
    rc = finalize_tables(grid_mode, B, N, H, W, C, pix_ws, &ft);
    if (rc) return rc;
    const int32_t* flag = mode_of(grid_mode) == IGS_GRID_AUTO ? grid_flag : nullptr;
    if (finalize_by_groups(ft.sup, B, N, ft.T))
        launch_finalize_listed<1>(FinalizeArgs{partial, ft.T, ft.T_alt, flag, ft.slots, ft.offsets, ft.overflow, ft.stamp, ft.sup,
                                               (N + 3) & ~3, N, C, C, scales,
                                               rotations, nullptr, alphas, eps, g_positions, g_scales, g_rotations,
                                               nullptr, g_alphas, g_colors},
                                  B, (hipStream_t)stream);
    else
        IGS_FINALIZE_LAUNCH(B, N, (k_bwd_finalize<true, kFT>),
                           (hipStream_t)stream, partial, ft.T, flag, ft.T_alt, ft.slots, ft.offsets, ft.overflow, ft.stamp,
                           (N + 3) & ~3, scales, rotations,
                           (const float*)nullptr, alphas, N, C, eps, g_positions,
                           g_scales, g_rotations, (float*)nullptr, g_alphas, g_colors);
    return launch_status();
}

int igs_gs2d_pack_feature(const float* gs_feature, const float* pos_offset, int B, int N, int C,
                          int C_kernel, float eps, float skip_weight, float skip_fraction, float* packed,
                          float* colors_out,
                          igs_stream_t stream) {
    if (!gs_feature || !packed || !colors_out) return IGS_ERR_NULL_POINTER;
    if (!shape_ok(B, N, 1, 1)) return IGS_ERR_BAD_SHAPE;
    if (C < 1 || C > C_kernel || !channels_compiled(C_kernel)) return IGS_ERR_BAD_CHANNELS;
    float limit;
    if (const int rc = limit_from_skip_weight(skip_weight, skip_fraction, &limit)) return rc;
    const int Np = (N + 3) & ~3;
    hipLaunchKernelGGL(k_pack_feature, dim3(ceil_div(Np, kThreads), B), dim3(kThreads), 0,
                       (hipStream_t)stream, gs_feature, pos_offset, N, Np, C, C_kernel,
                       rec_stride_of(C_kernel), eps, limit, skip_fraction, packed,
                       const_cast<float4*>(bins_of(packed, B, Np, rec_stride_of(C_kernel))),
                       const_cast<float*>(frecs_of(packed, B, Np, C_kernel)), frec_stride_of(C_kernel),
                       const_cast<float4*>(brecs_of(packed, B, Np, C_kernel)), colors_out);
    return launch_status();
}

int igs_gs2d_finalize_feature(const float* partial, const float* pix_ws, int grid_mode, const int32_t* grid_flag,
                              const float* gs_feature, int B, int N, int H, int W, int C,
                              int C_kernel, float eps, float* g_feature, igs_stream_t stream) {
    if (!partial || !gs_feature || !g_feature) return IGS_ERR_NULL_POINTER;
    int rc = mode_ok(grid_mode, grid_flag);
    if (rc) return rc;
    if (C < 1 || C > C_kernel || !channels_compiled(C_kernel)) return IGS_ERR_BAD_CHANNELS;
    FinalizeTables ft;
    rc = finalize_tables(grid_mode, B, N, H, W, C_kernel, pix_ws, &ft);
    if (rc) return rc;
    const int32_t* flag = mode_of(grid_mode) == IGS_GRID_AUTO ? grid_flag : nullptr;
    if (finalize_by_groups(ft.sup, B, N, ft.T))
        launch_finalize_listed<2>(FinalizeArgs{partial, ft.T, ft.T_alt, flag, ft.slots, ft.offsets, ft.overflow, ft.stamp, ft.sup,
                                               (N + 3) & ~3, N, C, C_kernel,
                                               gs_feature, nullptr, nullptr, nullptr, eps, g_feature, nullptr, nullptr,
                                               nullptr, nullptr, nullptr},
                                  B, (hipStream_t)stream);
    else
        IGS_FINALIZE_LAUNCH(B, N, (k_bwd_finalize_feature<kFT>),
                           (hipStream_t)stream, partial, ft.T, flag, ft.T_alt, ft.slots, ft.offsets, ft.overflow, ft.stamp,
                           (N + 3) & ~3, gs_feature,
                           N, C, C_kernel, eps, g_feature);
    return launch_status();
}

}  // extern "C"

// ------------------------------------------------------------------ KoLeo diversity loss
namespace {
// saved buffer: fn [B N Dp] | norm [B N] | nn_val [B N] | nn_idx [B N], each part 16-byte aligned
struct KoleoSaved {
    float* fn;
    float* norm;
    float* nn_val;
    int* nn_idx;
};

inline size_t koleo_rows_padded(long rows) { return (size_t)((rows + 3) & ~3L); }

KoleoSaved koleo_saved(void* saved, const igs_koleo_plan_t& p) {
    const long rows = (long)p.B * p.N;
    KoleoSaved s;
    s.fn = reinterpret_cast<float*>(saved);
    s.norm = s.fn + (size_t)rows * p.d_padded;
    s.nn_val = s.norm + koleo_rows_padded(rows);
    s.nn_idx = reinterpret_cast<int*>(s.nn_val + koleo_rows_padded(rows));
    return s;
}

int koleo_plan(int B, int N, int D, igs_koleo_plan_t* p) {
    if (!p) return IGS_ERR_NULL_POINTER;
    if (B <= 0 || B > 65535 || N < 2 || D <= 0 || D > (1 << 20)) return IGS_ERR_BAD_SHAPE;
    const int Dp = (D + 3) & ~3;
    if ((long)B * N > (1L << 28) || (long)B * N * Dp > (1L << 31)) return IGS_ERR_BAD_SHAPE;
    const int cus = device_cus() > 0 ? device_cus() : 256;
    int tile_rows, tile, S, per;
    if (Dp <= kKoleoMfmaMaxD) {
        // matrix-core kernel: a workgroup owns 128 query rows (32 per wave) and streams candidate tiles
        // of 32 rows; the candidates are split until there are four workgroups per compute unit
        tile_rows = 128;
        tile = 32;
        const int tiles = ceil_div(N, tile);
        S = ceil_div((long)IGS_KOLEO_WGS_PER_CU * cus, (long)ceil_div(N, tile_rows) * B);
        S = S < 1 ? 1 : (S > tiles ? tiles : S);
        per = ceil_div(tiles, S);
        S = ceil_div(tiles, per);
    } else {
        // similarity tiles of 128x64, unless one column tile per workgroup would leave most of the
        // device idle (then 64x64, then 32x32); after that enough workgroups for two per compute
        // unit, by splitting the columns
        const long t128 = ceil_div(N, 128), t64 = ceil_div(N, 64);
        // (128 rows pay only where the row tile is re-read from LDS at every step, Dp > kKoleoRegK)
        tile_rows = (Dp > kKoleoRegK && t128 * t64 * B >= 2L * cus) ? 128 : (t64 * t64 * B >= 2L * cus ? 64 : 32);
        tile = tile_rows == 32 ? 32 : 64;
        const int tiles = ceil_div(N, tile);
        const int row_tiles = ceil_div(N, tile_rows);
        S = ceil_div(2L * cus, (long)row_tiles * B);
        S = S < 1 ? 1 : (S > tiles ? tiles : S);
        per = ceil_div(tiles, S);
        S = ceil_div(tiles, per);
    }
    const long rows = (long)B * N;
    p->B = B;
    p->N = N;
    p->D = D;
    p->d_padded = Dp;
    p->tile_rows = tile_rows;
    p->tile = tile;
    p->splits = S;
    p->tiles_per_split = per;
    // backward: a wave owns bwd_rows rows.  More rows mean less scanning in total, but a wave
    // handles its rows one after the other, each a chain of dependent loads, so it takes four
    // waves per SIMD (4096 on the device) to hide that before rows are added.
    p->bwd_chunk = Dp < kKoleoBwdChunk ? Dp : kKoleoBwdChunk;
    int rw_max = kKoleoBwdLds / p->bwd_chunk;
    rw_max = rw_max > kKoleoBwdMaxRows ? kKoleoBwdMaxRows : rw_max;
    int rw = 1;
    while (rw * 2 <= rw_max && (long)B * N / (rw * 2) >= 16L * cus) rw *= 2;
    p->bwd_rows = rw;
    p->saved_bytes = ((size_t)rows * Dp + 3 * koleo_rows_padded(rows)) * sizeof(float);
    const size_t blocks = (size_t)ceil_div(rows, kThreads);
    p->scratch_bytes = ((blocks + 1) & ~(size_t)1) * sizeof(double) + (size_t)B * S * N * 2 * sizeof(float);
    return IGS_OK;
}
}  // namespace

extern "C" {
int igs_koleo_plan(int B, int N, int D, igs_koleo_plan_t* plan) { return koleo_plan(B, N, D, plan); }

int igs_koleo_forward(const float* features, int B, int N, int D, float* loss, void* saved,
                      size_t saved_bytes, void* scratch, size_t scratch_bytes, igs_stream_t stream) {
    if (!features || !loss || !saved || !scratch) return IGS_ERR_NULL_POINTER;
    igs_koleo_plan_t p;
    int rc = koleo_plan(B, N, D, &p);
    if (rc) return rc;
    if (saved_bytes < p.saved_bytes || scratch_bytes < p.scratch_bytes) return IGS_ERR_WORKSPACE;
    if (((uintptr_t)saved | (uintptr_t)scratch) & 15) return IGS_ERR_ALIGNMENT;
    const KoleoSaved sv = koleo_saved(saved, p);
    const long rows = (long)B * N;
    const int blocks = ceil_div(rows, kThreads);
    double* loss_part = reinterpret_cast<double*>(scratch);
    float* part_val = reinterpret_cast<float*>(loss_part + ((blocks + 1) & ~1));
    int* part_idx = reinterpret_cast<int*>(part_val + (size_t)B * p.splits * N);
    hipStream_t st = (hipStream_t)stream;
    hipLaunchKernelGGL(k_koleo_normalize, dim3(ceil_div(rows, kThreads / 64)), dim3(kThreads), 0, st,
                       features, rows, D, p.d_padded, sv.fn, sv.norm);
    const dim3 nn_grid(ceil_div(N, p.tile_rows), p.splits, B);
#define IGS_KOLEO_MFMA(KH)                                                                             \
    hipLaunchKernelGGL((k_koleo_nn_mfma<KH>), nn_grid, dim3(kThreads), 0, st, (const float*)sv.fn, N,   \
                       p.d_padded, p.tiles_per_split, part_val, part_idx)
#define IGS_KOLEO_NN(MR, MC, KN)                                                                       \
    hipLaunchKernelGGL((k_koleo_nn<MR, MC, KN>), nn_grid, dim3(kThreads), 0, st, (const float*)sv.fn, N, \
                       p.d_padded, p.tiles_per_split, part_val, part_idx)
#define IGS_KOLEO_NN_K(KN)                                           \
    do {                                                             \
        if (p.tile_rows == 128 && KN == 0) IGS_KOLEO_NN(8, 4, 0);    \
        else if (p.tile_rows == 64) IGS_KOLEO_NN(4, 4, KN);          \
        else IGS_KOLEO_NN(2, 2, KN);                                 \
    } while (0)
    if (p.d_padded <= kKoleoMfmaMaxD) {  // MFMAs per candidate tile: half the (padded) row length, rounded up
        const int kh = p.d_padded / 2;
        if (kh <= 2) IGS_KOLEO_MFMA(2);
        else if (kh <= 4) IGS_KOLEO_MFMA(4);
        else if (kh <= 6) IGS_KOLEO_MFMA(6);
        else if (kh <= 8) IGS_KOLEO_MFMA(8);
        else if (kh <= 12) IGS_KOLEO_MFMA(12);
        else if (kh <= 16) IGS_KOLEO_MFMA(16);
        else if (kh <= 24) IGS_KOLEO_MFMA(24);
        else IGS_KOLEO_MFMA(32);
    } else
    switch (p.d_padded <= kKoleoRegK ? p.d_padded : 0) {
        case 4: IGS_KOLEO_NN_K(4); break;
        case 8: IGS_KOLEO_NN_K(8); break;
        case 12: IGS_KOLEO_NN_K(12); break;
        case 16: IGS_KOLEO_NN_K(16); break;
        default: IGS_KOLEO_NN_K(0); break;
    }
#undef IGS_KOLEO_MFMA
#undef IGS_KOLEO_NN_K
#undef IGS_KOLEO_NN
    hipLaunchKernelGGL(k_koleo_combine, dim3(blocks), dim3(kThreads), 0, st, (const float*)part_val,
                       (const int*)part_idx, (const float*)sv.norm, B, N, p.splits, sv.nn_val, sv.nn_idx,
                       loss_part);
    hipLaunchKernelGGL(k_koleo_sum, dim3(1), dim3(kThreads), 0, st, (const double*)loss_part, blocks,
                       1.0 / (double)rows, loss);
    return launch_status();
}

int igs_koleo_backward(const void* saved, size_t saved_bytes, const float* grad_loss, int B, int N,
                       int D, float* grad_features, igs_stream_t stream) {
    if (!saved || !grad_loss || !grad_features) return IGS_ERR_NULL_POINTER;
    igs_koleo_plan_t p;
    int rc = koleo_plan(B, N, D, &p);
    if (rc) return rc;
    if (saved_bytes < p.saved_bytes) return IGS_ERR_WORKSPACE;
    if ((uintptr_t)saved & 15) return IGS_ERR_ALIGNMENT;
    const KoleoSaved sv = koleo_saved(const_cast<void*>(saved), p);
    hipLaunchKernelGGL(k_koleo_bwd, dim3(ceil_div(N, p.bwd_rows), B), dim3(64),
                       (size_t)p.bwd_rows * p.bwd_chunk * sizeof(float), (hipStream_t)stream,
                       (const float*)sv.fn, (const float*)sv.norm, (const int*)sv.nn_idx, grad_loss, B, N, D,
                       p.d_padded, p.bwd_rows, p.bwd_chunk, grad_features);
    return launch_status();
}

}  // extern "C"
