/* igs_hip.h -- C ABI of libigs_hip.so: 2-D Gaussian splatting forward/backward for
 * AMD MI355X (gfx950).
 *
 * This is the boundary a host framework binds (ctypes / cffi / pybind / dlopen).  Every
 * entry point takes plain device pointers and sizes; the library never allocates, frees or
 * keeps a pointer, never synchronises the device, and launches on the stream it is given.
 * All tensors are fp32 and dense/contiguous unless a stride argument says otherwise.
 * Return value: 0 on success, a negative igs_status for a rejected argument, or a positive
 * hipError_t if a launch failed.  No C++ exception crosses this boundary.
 *
 * Reference interfaces replaced (paths relative to the KohakuBlueleaf/IGS checkout):
 *   - the `.apply(x, y, position, cov_inv_00, cov_inv_01, cov_inv_11, alphas, colors, eps)`
 *     operator, forward + backward: src/igs/gs2d.py:47-262, :265-465,
 *     src/igs/gs_triton.py:408-640, src/igs/gs_triton_chunked.py:543-924;
 *   - the covariance-inverse preamble of `render`: src/igs/gs2d.py:548-580.
 */
#ifndef IGS_HIP_H
#define IGS_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define IGS_ABI_VERSION 8
#define IGS_MAX_CHANNELS 16
/* Size of the per-device static scratch array behind igs_gs2d_forward_static_ws. */
#define IGS_STATIC_SCRATCH_BYTES (64u << 20)

typedef void *igs_stream_t; /* a hipStream_t */

typedef enum igs_status {
    IGS_OK = 0,
    IGS_ERR_NULL_POINTER = -1,
    IGS_ERR_BAD_SHAPE = -2,      /* a dimension <= 0 or too large: B <= 65535, N <= 2^24,
                                    B*N <= 2^28, H*W <= 2^28 */
    IGS_ERR_BAD_CHANNELS = -3,   /* C outside 1..IGS_MAX_CHANNELS */
    IGS_ERR_WORKSPACE = -4,      /* a workspace is smaller than igs_gs2d_plan says */
    IGS_ERR_BAD_MODE = -5,       /* unknown grid mode */
    IGS_ERR_NO_DEVICE = -6,      /* no usable HIP device */
    IGS_ERR_ALIGNMENT = -7,      /* a buffer that must be 16-byte aligned is not */
    IGS_ERR_STATIC_SCRATCH = -8, /* igs_gs2d_forward_static_ws: the plan's fwd_ws_bytes exceeds
                                    IGS_STATIC_SCRATCH_BYTES */
    IGS_ERR_STATIC_BUSY = -10,   /* igs_gs2d_forward_static_ws: the previous call on this device, made on
                                    another stream, has not finished with the one scratch array */
    IGS_ERR_BAD_SKIP_WEIGHT = -9 /* a pack call's skip_weight or skip_fraction is negative, NaN
                                    or >= 1 */
} igs_status;

/* How the pixel coordinates are described.
 * x(b,h,w) = x[b*sxb + h*sxh + w*sxw], y likewise with (syb, syh, syw); strides are in
 * elements and may be 0 (expanded tensors).
 *   IGS_GRID_GENERAL   : arbitrary per-pixel coordinates (what the reference operator
 *                        accepts, src/igs/gs2d.py:82-83).
 *   IGS_GRID_SEPARABLE : the caller guarantees x does not depend on h and y does not
 *                        depend on w (every linspace/meshgrid grid, e.g. xy_grid,
 *                        src/igs/gs2d.py:503-522).  sxh and syw are then ignored and the
 *                        kernels factor the quadratic form by rows/columns.
 *   IGS_GRID_AUTO      : decided on the device, without a host synchronisation: the caller
 *                        runs igs_gs2d_grid_classify once into a 4-byte flag and passes that
 *                        flag to every later call; both kernel variants are enqueued and the
 *                        flag selects the one that does the work (the other exits at once).
 *                        Workspace sizes are the larger of the two variants'.
 * Entry points take `grid_flag` (device int32, 1 = separable); it is only read in AUTO mode
 * and may be NULL otherwise.
 *
 * The `grid_mode` argument of an entry point carries the igs_grid_mode in its low byte and may
 * have igs_option bits OR-ed in above it (testing aids; they change no buffer size, and unknown
 * bits are rejected with IGS_ERR_BAD_MODE).  A backward and its finalize call must get the same
 * IGS_OPT_BIN_LEVELS_* bits.
 */
typedef enum igs_grid_mode {
    IGS_GRID_GENERAL = 0,
    IGS_GRID_SEPARABLE = 1,
    IGS_GRID_AUTO = 2
} igs_grid_mode;

typedef enum igs_option {
    IGS_OPT_NO_CULL = 0x100,      /* separable grids: list every Gaussian for every pixel tile
                                     (nothing is skipped): the reference point for checking what
                                     skipping changes */
    IGS_OPT_BIN_LEVELS_1 = 0x200, /* build the per-tile Gaussian lists in one level ...           */
    IGS_OPT_BIN_LEVELS_2 = 0x400, /* ... or through super-tiles of 4 x 4 tiles, whatever the size;
                                     without either bit the library chooses by tiles x N          */
    IGS_OPT_LISTS_BUILT = 0x800   /* igs_gs2d_backward_reduce / igs_gs2d_backward /
                                     igs_gs2d_backward_with_grid only: the tile lists and slot
                                     tables are in these workspaces already
                                     (igs_gs2d_forward_train built them for this packed
                                     buffer and these grids); do not build them again            */
} igs_option;

/* Launch plan and workspace sizes for one problem shape (filled by igs_gs2d_plan).  In AUTO
 * mode the geometry fields describe the separable variant. */
typedef struct igs_gs2d_plan_t {
    int32_t B, N, H, W, C;
    int32_t rec_stride;      /* floats per packed Gaussian record                          */
    int32_t n_padded;        /* records per image in the packed buffer (N rounded up to 4) */
    int32_t w_padded;        /* separable: pixel-record columns per row (W rounded up to 8)*/
    int32_t hw_padded;       /* general: pixel records per image (H*W rounded up to 4)     */
    int32_t fwd_split;       /* number of Gaussian-range splits of the forward (>= 1)      */
    int32_t fwd_n_per_split; /* records per split (multiple of 4)                          */
    int32_t bwd_tiles;       /* pixel tiles T per image of the backward partial buffer     */
    int32_t bwd_per_tile;    /* rows (separable) or pixels (general) per backward tile     */
    int32_t pix_stride;      /* floats per pixel record of the backward prologue           */
    uint64_t packed_bytes;   /* packed Gaussian buffer: records, then one bin record (8
                                floats: reach box and quadratic form, what the tile lists
                                are built from) per record, then the call's skip settings
                                (4 floats) and an all-zero record (28 floats), then the
                                separable kernels' own records (forward: roundup4(10+C)
                                floats, none for C > 8; backward: 4 floats):
                                (B*n_padded*(rec_stride+8+sep) + 32)*4                     */
    uint64_t fwd_ws_bytes;   /* forward scratch: split partials (fwd_split > 1) and, on
                                separable grids, the per-tile Gaussian lists (plus those
                                of the super-tiles when there are 32 tiles or more)         */
    uint64_t pix_bytes;      /* backward scratch: per-pixel records and, on separable
                                grids, the backward's tables: the Gaussian lists as above,
                                the slot tables of the tiles (and super-tiles), the tiles'
                                first records in the partial-sum array, an overflow flag    */
    uint64_t partial_bytes;  /* backward partial sums when every Gaussian is stored for
                                every tile, B*T*(6+C)*N*4: what general grids need, and an
                                upper bound of what the separable backward needs, which is
                                (6+C)*4 bytes per listed (Gaussian, tile) entry, see
                                igs_gs2d_forward_train                                     */
    int32_t fwd_tiles;       /* separable: pixel tiles per image of the forward            */
    int32_t bwd_tiles_x;     /* separable: column bands of the backward tiles              */
    int32_t bwd_tile_w;      /* separable: columns per band                                */
    int32_t lists_shared;    /* separable: the backward's tiles are the forward's wave
                                rectangles, so igs_gs2d_forward_train can build one
                                set of tile lists for both passes                           */
} igs_gs2d_plan_t;

int igs_abi_version(void);
const char *igs_status_string(int status);

/* Shape -> launch plan + workspace sizes.  Pure host arithmetic apart from a cached
 * query of the current device's compute-unit count.  grid_mode is an igs_grid_mode. */
int igs_gs2d_plan(int B, int N, int H, int W, int C, int grid_mode, igs_gs2d_plan_t *plan);

/* Device-side test whether the grids are separable (bitwise: x(b,h,w) == x(b,0,w) and
 * y(b,h,w) == y(b,h,0)); writes 1 or 0 to *grid_flag.  No counterpart in the reference,
 * whose kernels always read per-pixel coordinates (src/igs/gs_triton.py:113-114). */
int igs_gs2d_grid_classify(const float *x, const float *y, const int64_t grid_strides[6], int B,
                           int H, int W, int32_t *grid_flag, igs_stream_t stream);

/* tolerance * eps / (2 N) (0 when eps <= 0 or tolerance <= 0), capped at 0.5: the skip_weight, and
 * with eps = 1 the skip_fraction, with which what the kernels skip changes every output element
 * by at most tolerance * max|colors| (see igs_gs2d_pack_covinv).  The host side of this build
 * passes tolerance = 1e-7 against the 1e-6 + 1e-5 |ref| that the forward is held to.  Pure host
 * arithmetic; no counterpart in the reference, which evaluates every pair. */
float igs_gs2d_skip_weight(int N, float eps, float tolerance);

/* Pack per-Gaussian parameters for the kernels (operator level: the caller already has
 * the inverse covariance).  position [B,N,2]; cov_inv_00/01/11 [B,N]; alphas [B,N];
 * colors [B,N,C]; packed: plan.packed_bytes, 16-byte aligned.  Replaces nothing in the
 * reference (its kernels read the tensors directly); it exists so the hot loops read one
 * record.  Behind the records the buffer holds one bin record per Gaussian (its "reach box" and
 * quadratic form) and the call's skip settings.  On separable grids the forward and the backward skip, per pixel tile (and the forward
 * per wave of rows), the Gaussians whose box misses the tile or whose ellipse does not reach the
 * tile's coordinate rectangle (the reference evaluates every pair:
 * src/igs/gs_triton_chunked.py:100-200).  What may be skipped is set by skip_weight w and
 * skip_fraction f, both in [0, 1):
 *   w = f = 0: only pairs whose exponential is exactly 0 in fp32.  The order of the other terms
 *     is kept, so results equal those of not skipping bit for bit while the forward runs one
 *     Gaussian split (plan.fwd_split == 1), and to fp32 rounding otherwise, where a tile's list
 *     rather than the index range is cut into the splits.
 *   otherwise: per pixel tile (per wave rectangle in the forward), a set of Gaussians is left out
 *     whose largest terms on the tile add up to at most N (w + f S).  A Gaussian's largest term
 *     is exp(-q/2) max(1, |alpha|) at the point of the tile's coordinate rectangle where q is
 *     smallest, so it bounds both its weight alpha e and the bare exponential (which the gradient
 *     of alpha sums) on every pixel of the tile.  S is a lower bound of the tile's denominators:
 *     the sum, over the Gaussians whose box meets the tile, of the least weight each has on it (0
 *     if one of them has a negative or non-finite alpha).  Gaussians whose largest term is below w
 *     are always left out; of the others the lightest are, by whole classes of half a binade of
 *     weight, as far as what remains of the allowance goes.  Per pixel the skipped weights then add
 *     up to at most N (w + f S): den changes by at most that and an output element by at most
 *     N (w + f S) (max|colors| + |out|) / (den + eps) <= 2 N max|colors| max(w / eps, f) for
 *     den >= S; a per-Gaussian gradient sum misses, for a pixel of a tile the Gaussian is not
 *     listed for, a term of at most N (w + f S) |G| |moment|, |G| <= 2 max|colors| |grad_out| /
 *     (den + eps).  igs_gs2d_skip_weight gives w and f for a wanted bound.
 * Records with a non-finite field or a cov_inv that is not positive definite are never skipped;
 * with IGS_OPT_NO_CULL in a forward / backward call's grid_mode nothing is.
 * Large problems (tiles x N >= 6e6) build the per-tile lists in two levels (super-tiles of
 * 4 x 4 tiles first); IGS_OPT_BIN_LEVELS_1|2 forces one or two.  With w = f = 0 the lists and
 * the forward do not depend on it; otherwise a tile settles what it leaves out from the
 * candidates it sees, so the lists may differ within the same bound.  The finalize kernels add
 * the tiles in another order under two levels, so gradients agree to fp32 rounding. */
int igs_gs2d_pack_covinv(const float *position, const float *cov_inv_00, const float *cov_inv_01,
                         const float *cov_inv_11, const float *alphas, const float *colors,
                         int B, int N, int C, float skip_weight, float skip_fraction,
                         float *packed, igs_stream_t stream);

/* Same, from scales [B,N,2] and rotations [B,N]: closed form of
 * (R S S^T R^T + eps I)^-1, replacing src/igs/gs2d.py:548-580. */
int igs_gs2d_pack_scale_rot(const float *positions, const float *scales, const float *rotations,
                            const float *alphas, const float *colors, int B, int N, int C,
                            float eps, float skip_weight, float skip_fraction, float *packed,
                            igs_stream_t stream);

/* Forward: out [B,C,H,W] = sum_n w_n c_n / (sum_n w_n + eps), den [B,H,W] = sum_n w_n.
 * Replaces the forward of src/igs/gs2d.py:68-144 / src/igs/gs_triton_chunked.py:551-680.
 * grid_strides = {sxb, sxh, sxw, syb, syh, syw}.  ws: scratch of plan.fwd_ws_bytes, 16-byte
 * aligned (may be NULL when that is 0); its contents mean nothing after the call. */
int igs_gs2d_forward(const float *packed, const float *x, const float *y,
                     const int64_t grid_strides[6], int grid_mode, const int32_t *grid_flag, int B,
                     int N, int H, int W, int C, float eps, float *out, float *den, void *ws,
                     size_t ws_bytes, igs_stream_t stream);

/* igs_gs2d_forward without a workspace argument and without any allocation.  It has no
 * counterpart in the reference; it is for callers that cannot allocate device memory around the
 * call: code under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc.
 * The forward's scratch (split partials, per-tile Gaussian lists) lives in a static device array
 * of IGS_STATIC_SCRATCH_BYTES (64 MiB) that every GPU the library runs on holds until the process
 * ends; problems whose plan.fwd_ws_bytes is larger are rejected with IGS_ERR_STATIC_SCRATCH
 * (B=1, N=2048, 256x256, C=3 needs 32.5 MiB; the 16-image headline shape needs 160 MiB and must use
 * igs_gs2d_forward).  Same kernels, same launch plan and bit-identical results as
 * igs_gs2d_forward.  All calls on one GPU share that GPU's array: calls that overlap in time on
 * one GPU (two streams, two threads) race on it; nothing in it has to start at zero and its
 * contents mean nothing after the call.  A cheap guard catches the common case: a call made on
 * another stream than the previous one while that one's work has not finished (an event recorded
 * behind each call, queried without waiting) returns IGS_ERR_STATIC_BUSY instead of running; calls
 * on one stream are ordered by the stream and never refused.  The guard is off while the stream
 * is being captured into a graph (a replayed graph's overlap with other work stays the caller's
 * to exclude).  The first call on a device resolves the array's device
 * address (hipGetSymbolAddress, which may load the code object there): make that call outside
 * graph capture, with that device current. */
int igs_gs2d_forward_static_ws(const float *packed, const float *x, const float *y,
                               const int64_t grid_strides[6], int grid_mode,
                               const int32_t *grid_flag, int B, int N, int H, int W, int C,
                               float eps, float *out, float *den, igs_stream_t stream);

/* The forward of a training step (a backward on the same packed buffer and grids follows): as
 * igs_gs2d_forward, and on separable grids the backward's tables (per-tile Gaussian lists, slot
 * tables, the tiles' first records in the partial-sum array) are built as well, in pix_ws
 * (plan.pix_bytes; they depend on the packed buffer and the grids only).  Where plan.lists_shared
 * says that the backward's pixel tiles are the forward's wave rectangles, that one set of lists
 * serves both passes (one binning per step instead of two); elsewhere (small problems, whose
 * backward tiles have fewer rows) the backward's lists are made beside the forward's own by the
 * same launch.  The backward calls on the same pix_ws then get IGS_OPT_LISTS_BUILT in their
 * grid_mode (the prologue writes other parts of pix_ws).
 * listed_total, when not NULL, receives the number of listed (Gaussian, tile) entries, i.e. the
 * records the separable backward will store: its partial-sum array then needs listed_total *
 * (6+C) * 4 bytes (at least one record) instead of plan.partial_bytes.  The kernel writes it, so it
 * must be memory the device can write (device memory, or pinned host memory that the caller reads
 * after the stream reaches this point).
 * The output matches igs_gs2d_forward's up to what the skip tolerance allows (a tile settles what
 * it leaves out by itself, and the tiles of the two binnings need not be the same); bit for bit
 * with skip_weight = skip_fraction = 0 and one Gaussian split.  No counterpart in the reference,
 * which evaluates every pair (src/igs/gs_triton_chunked.py:100-200). */
int igs_gs2d_forward_train(const float *packed, const float *x, const float *y,
                           const int64_t grid_strides[6], int grid_mode, const int32_t *grid_flag,
                           int B, int N, int H, int W, int C, float eps, float *out, float *den,
                           void *ws, size_t ws_bytes, float *pix_ws, size_t pix_bytes,
                           int64_t *listed_total, igs_stream_t stream);

/* Backward, stage 1: per-pixel prologue, g^ = grad_out/(den+eps), s = <g^, out>, written
 * as one record per pixel into pix_ws (plan.pix_bytes).  Replaces the per-image pre-pass of
 * the reference backward, src/igs/gs2d.py:175-177 (which also mutates its inputs; this does
 * not).  out, grad_out [B,C,H,W]; den [B,H,W]. */
int igs_gs2d_backward_prologue(const float *x, const float *y, const int64_t grid_strides[6],
                               int grid_mode, const int32_t *grid_flag, const float *out,
                               const float *den, const float *grad_out, int B, int N, int H, int W,
                               int C, float eps, float *pix_ws, size_t pix_bytes,
                               igs_stream_t stream);

/* Backward, stage 2: the recomputing per-Gaussian reduction over pixel tiles into `partial`.
 * Replaces the Gaussian loop of the reference backward, src/igs/gs2d.py:180-246 /
 * src/igs/gs_triton.py:159-405.  colors [B,N,C].  pix_ws is the buffer stage 1 filled (16-byte
 * aligned); on separable grids this stage also writes its tables (per-tile Gaussian lists, slot
 * tables, record offsets) behind the pixel records in it, unless IGS_OPT_LISTS_BUILT says that
 * igs_gs2d_forward_train did.
 * partial: general grids store one record of 6+C sums for every Gaussian and tile, [B,T,N,6+C]
 * (plan.partial_bytes, required).  The separable backward stores the records of the listed
 * (Gaussian, tile) entries only, tile after tile: partial_bytes may be as small as their number
 * (igs_gs2d_forward_train's listed_total) * (6+C) * 4, at least one record; plan.partial_bytes
 * always suffices.  Where partial_bytes does not hold them, nothing is stored for the tiles that
 * do not fit and the flag in pix_ws is raised, upon which the finalize calls return NaN for every
 * gradient (no status: nothing here waits for the device).  In AUTO mode plan.partial_bytes is
 * required. */
int igs_gs2d_backward_reduce(const float *packed, const float *colors, const float *y,
                             const int64_t grid_strides[6], int grid_mode, const int32_t *grid_flag,
                             int B, int N, int H, int W, int C, float *pix_ws,
                             size_t pix_bytes, float *partial, size_t partial_bytes,
                             igs_stream_t stream);

/* Stages 1 and 2 in one call. */
int igs_gs2d_backward(const float *packed, const float *colors, const float *x, const float *y,
                      const int64_t grid_strides[6], int grid_mode, const int32_t *grid_flag,
                      const float *out, const float *den, const float *grad_out, int B, int N,
                      int H, int W, int C, float eps, float *pix_ws, size_t pix_bytes,
                      float *partial, size_t partial_bytes, igs_stream_t stream);

/* Stages 1 and 2 plus the gradients w.r.t. the pixel coordinates g_x, g_y [B,H,W] (grad_x /
 * grad_y of the reference backward, src/igs/gs2d.py:222-231, :249-250, which always computes
 * them) in one call.  On general grids the per-pixel sums are formed inside the per-Gaussian
 * reduction (one exponential per pair instead of two) into grid_ws
 * (igs_gs2d_grid_workspace_bytes, 8-byte aligned) and added in a fixed order; on separable
 * grids this equals igs_gs2d_backward followed by igs_gs2d_backward_grid, and with
 * IGS_GRID_SEPARABLE grid_ws is not used and may be NULL. */
size_t igs_gs2d_grid_workspace_bytes(int B, int N, int H, int W, int C);
int igs_gs2d_backward_with_grid(const float *packed, const float *colors, const float *x,
                                const float *y, const int64_t grid_strides[6], int grid_mode,
                                const int32_t *grid_flag, const float *out, const float *den,
                                const float *grad_out, int B, int N, int H, int W, int C, float eps,
                                float *pix_ws, size_t pix_bytes, float *partial,
                                size_t partial_bytes, void *grid_ws, size_t grid_ws_bytes,
                                float *g_x, float *g_y, igs_stream_t stream);

/* Optional backward output: gradients w.r.t. the pixel coordinates, g_x, g_y [B,H,W]
 * (grad_x / grad_y of the reference backward, src/igs/gs2d.py:222-231, :249-250; the Triton
 * backward accumulates them with atomics, src/igs/gs_triton.py:365-366).  Independent of the
 * other backward stages: reads packed, out, den, grad_out; needs no workspace.  Only run
 * when the caller wants these gradients. */
int igs_gs2d_backward_grid(const float *packed, const float *x, const float *y,
                           const int64_t grid_strides[6], const float *out, const float *den,
                           const float *grad_out, int B, int N, int H, int W, int C, float eps,
                           float *g_x, float *g_y, igs_stream_t stream);

/* Backward, stage 3 (operator level): fixed-order sum of the tile partials and the
 * gradients of the operator inputs (the tail of src/igs/gs2d.py:207-246, :252-262).  The
 * shape and grid mode must be those given to igs_gs2d_backward (they fix the tile count).
 * Any output pointer may be NULL (not wanted).  pix_ws: the backward's pixel workspace, whose
 * tables say where a Gaussian's records are (separable and AUTO modes; may be NULL with
 * IGS_GRID_GENERAL).
 * g_position [B,N,2]; g_cov_inv_* [B,N]; g_alphas [B,N]; g_colors [B,N,C]. */
int igs_gs2d_finalize_covinv(const float *partial, const float *pix_ws, int grid_mode,
                             const int32_t *grid_flag,
                             const float *cov_inv_00, const float *cov_inv_01,
                             const float *cov_inv_11, const float *alphas, int B, int N, int H,
                             int W, int C, float *g_position, float *g_cov_inv_00,
                             float *g_cov_inv_01, float *g_cov_inv_11, float *g_alphas,
                             float *g_colors, igs_stream_t stream);

/* Backward, stage 3 (function level): as above plus the chain rule through the closed-form
 * covariance inverse to scales [B,N,2] and rotations [B,N] (the autograd of
 * src/igs/gs2d.py:548-580). */
int igs_gs2d_finalize_scale_rot(const float *partial, const float *pix_ws, int grid_mode,
                                const int32_t *grid_flag,
                                const float *scales, const float *rotations, const float *alphas,
                                int B, int N, int H, int W, int C, float eps, float *g_positions,
                                float *g_scales, float *g_rotations, float *g_alphas,
                                float *g_colors, igs_stream_t stream);

/* Module head fused into pack / finalize (replaces the split + activations of the module's
 * forward, src/igs/gs2d.py:635-644 and :673-675, and their autograd).
 * gs_feature [B,N,6+C] rows: px, py, log_s0, log_s1, theta, opacity logit (unused), c_0..;
 * scales = exp(log_s) + eps, alpha = 1.  pos_offset [B,N,2] is added to the positions when not
 * NULL (pos_map_offset, src/igs/gs2d.py:654-667).  C_kernel is the compiled channel count
 * (>= C) the other calls are made with; colors_out [B,N,C_kernel] receives the zero-padded raw
 * colours for igs_gs2d_backward.  g_feature [B,N,6+C] gets d L / d gs_feature (0 for the
 * opacity logit); d L / d pos_offset equals its first two columns.  skip_weight, skip_fraction:
 * as in igs_gs2d_pack_covinv. */
int igs_gs2d_pack_feature(const float *gs_feature, const float *pos_offset, int B, int N, int C,
                          int C_kernel, float eps, float skip_weight, float skip_fraction,
                          float *packed, float *colors_out, igs_stream_t stream);
int igs_gs2d_finalize_feature(const float *partial, const float *pix_ws, int grid_mode,
                              const int32_t *grid_flag,
                              const float *gs_feature, int B, int N, int H, int W, int C,
                              int C_kernel, float eps, float *g_feature, igs_stream_t stream);

/* Fit step (single-image fitting loop, scripts/2dgs_img_comp.py:186-193 and :219-232):
 * render -> loss -> backward -> AdamW without leaving the library between the stages.
 *
 * igs_gs2d_backward_prologue_mse is igs_gs2d_backward_prologue with the upstream gradient of
 * loss = mean((out - target)^2) (F.mse_loss, scripts/2dgs_img_comp.py:133) formed inside the
 * per-pixel pass: g = 2 (out - target) / (B C_real H W).  out and target are [B,C,H,W] with the
 * compiled channel count C; channels C_real..C-1 must be zero in both.  The loss value is
 * written to loss[0] (device; fixed-order sum, bit-reproducible).  loss_ws needs
 * igs_gs2d_mse_workspace_bytes(B,H,W) bytes.  Follow with igs_gs2d_backward_reduce. */
size_t igs_gs2d_mse_workspace_bytes(int B, int H, int W);
int igs_gs2d_backward_prologue_mse(const float *x, const float *y, const int64_t grid_strides[6],
                                   int grid_mode, const int32_t *grid_flag, const float *out,
                                   const float *den, const float *target, int C_real, int B, int N,
                                   int H, int W, int C, float eps, float *pix_ws, size_t pix_bytes,
                                   float *loss_ws, size_t loss_ws_bytes, float *loss,
                                   igs_stream_t stream);

/* Position regulariser of the fit loop, scripts/2dgs_img_comp.py:224-228:
 * position_penalty = mean(relu(|position| - 1)), added to the loss with a weight (0.01 there).
 * gs_feature is `rows` rows of `row_floats` floats whose first two are the position; `count` is
 * the number of position elements the mean runs over (2 x the number of all Gaussians of the
 * model, also when only a prefix of them is passed).  Adds weight * sign(p) [|p| > 1] / count to
 * the position columns of g_feature (same layout; call after igs_gs2d_finalize_feature, before
 * igs_adamw_step) and, when loss is not NULL, weight * mean to loss[0] (device; fixed-order sum). */
int igs_gs2d_position_penalty(const float *gs_feature, int64_t rows, int row_floats, float weight,
                              int64_t count, float *g_feature, float *loss, igs_stream_t stream);

/* One torch.optim.AdamW step (amsgrad off; the optimiser of scripts/2dgs_img_comp.py:186-193)
 * over a flat block of `count` floats, in place:
 *   p *= 1 - lr wd;  m += (g - m)(1 - beta1);  v = beta2 v + (1 - beta2) g^2;
 *   p -= lr / (1 - beta1^t) * m / (sqrt(v) / sqrt(1 - beta2^t) + eps).
 * state is 8 floats of device memory {lr, t, 1 - beta1^t, sqrt(1 - beta2^t), ticket, 0, 0, 0}: the
 * caller zeroes it before the first step and writes lr; every call increments t on the device (the
 * last workgroup to finish does, through the integer ticket, which is zero again when the call is
 * done), so a captured graph of the call advances on each replay.  One launch. */
int igs_adamw_step(float *param, const float *grad, float *exp_avg, float *exp_avg_sq,
                   int64_t count, float *state, float beta1, float beta2, float eps,
                   float weight_decay, igs_stream_t stream);

/* ---- KoLeo diversity loss (src/igs/reg.py:5-40) ---------------------------------------------
 * loss = mean over the B*N rows of relu(max_{j != i} cos(x_i, x_j) + 1), features [B,N,D] fp32
 * contiguous.  The reference normalises the rows, forms the [B,N,N] similarity matrix with bmm,
 * fills its diagonal with -inf and takes the row maxima; these entry points compute the same
 * maxima tile by tile and never hold the matrix.  Equal similarities resolve to the lowest
 * column index; every sum has a fixed order (results are bit-reproducible).  N >= 2 (the
 * reference returns a constant 0 for N <= 1, src/igs/reg.py:19-20: callers handle that case). */
typedef struct igs_koleo_plan_t {
    int32_t B, N, D;
    int32_t d_padded;        /* floats per normalised row (D rounded up to 4)                 */
    int32_t tile_rows;       /* rows a workgroup searches for: 128, 64 or 32 (by problem size) */
    int32_t tile;            /* candidate rows per similarity tile: 64 or 32                   */
    int32_t splits;          /* column splits of the similarity tiles (>= 1)                  */
    int32_t tiles_per_split; /* column tiles per split                                         */
    int32_t bwd_rows;        /* rows per wave of the backward                                  */
    int32_t bwd_chunk;       /* feature dimensions per pass of the backward                    */
    uint64_t saved_bytes;    /* kept from forward to backward: normalised rows, norms, nearest
                                similarity and neighbour index per row                        */
    uint64_t scratch_bytes;  /* forward only: per-split maxima, per-workgroup loss sums       */
} igs_koleo_plan_t;

int igs_koleo_plan(int B, int N, int D, igs_koleo_plan_t *plan);

/* Forward: writes *loss (one float of device memory) and fills `saved` (plan.saved_bytes,
 * 16-byte aligned) for the backward.  Replaces src/igs/reg.py:22-37. */
int igs_koleo_forward(const float *features, int B, int N, int D, float *loss, void *saved,
                      size_t saved_bytes, void *scratch, size_t scratch_bytes, igs_stream_t stream);

/* Backward: grad_features [B,N,D] = grad_loss[0] * d loss / d features from the forward's
 * `saved` buffer (what autograd derives from src/igs/reg.py:22-37: the gradient reaches a row
 * through its own nearest neighbour and through the rows whose nearest neighbour it is, then
 * through the normalisation).  grad_loss is one float of device memory. */
int igs_koleo_backward(const void *saved, size_t saved_bytes, const float *grad_loss, int B, int N,
                       int D, float *grad_features, igs_stream_t stream);

#ifdef __cplusplus
}
#endif
#endif /* IGS_HIP_H */
