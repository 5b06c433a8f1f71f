// igs_forward.h -- forward kernels: LDS record streaming, separable and general grids, split combine.
// Included by igs_gs2d.hip inside its anonymous namespace (one translation unit).
#pragma once

// ----------------------------------------------------------------------------- forward
struct FwdArgs {
    const float* packed;  // [B][Np][RS]
    const float* frecs;   // separable kernels: their forward records [B][Np][frec_stride_of(C)]
    const float* zero_rec;  // an all-zero record behind the packed buffer's skip settings
    const float* x;
    const float* y;
    long sxb, sxh, sxw, syb, syh, syw;
    int B, Np, H, W;
    int n_per_split, S;  // n_per_split % 4 == 0
    int tiles_x, tiles_y, total_tiles, wx, wcols;  // shared lists: wx waves of wcols columns side by side
    float eps;
    float* out;
    float* den;
    float* part;  // [S][B][C+1][HW] when S > 1
    const int* counts;  // separable: Gaussians listed per tile [B][tiles], or per wave rectangle, row after row over the tiles' extent [B][4 tiles]
    const int* lists;   // separable: their indices [B][lists][Np]
    int list_img, list_row;  // lists per image and per row of rectangles (tiles) in that numbering
    const int* flag;  // AUTO grid mode: run only if *flag == want (nullptr: always run)
    int want;
    float ramp;  // separable: how far the parts of a list differ in length (kSplitRamp, or 0 when all waves are resident at once)
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
    float ylo, yhi;  // y range of the reach box (records with two spare floats only)
};

// whether a record of C channels has room for the y range of the reach box
__host__ __device__ constexpr bool rec_has_yrange(int C) { return rec_stride_of(C) >= 8 + C; }
// The separable forward variants whose lanes hold 16 or 8 rows (C <= 8) give every wave a Gaussian list
// of its own (kWaveCols columns x 64 P / kWaveCols rows); the four waves of a workgroup stream theirs
// independently: no wave waits for another at a chunk boundary, and none reads records it then skips.  With 4 rows per
// wave (C = 16) the tile of four waves is small already and the lists of single waves cost the
// binning more than the forward gains (B=4, N=32768, 384x640: 3.25 -> 3.73 ms): that variant streams
// one list to four waves, and a wave tests the reach box's y range against its own rows.
// Columns of a wave's rectangle where every wave has a list of its own: 32 columns x 2 P rows (32 x 32
// pixels for C <= 3) are reached by fewer Gaussians than 64 x P (B=16 N=8192 256x256: forward 1.16 ->
// 1.10 ms; B=1 N=16384 512x512: 0.209 -> 0.193 ms).
#ifndef IGS_FWD_WAVE_COLS
#define IGS_FWD_WAVE_COLS 32
#endif
constexpr int kWaveCols = IGS_FWD_WAVE_COLS;
static_assert(kWaveCols == 64 || kWaveCols == 32, "wave rectangle");
#ifndef IGS_FWD_WAVE_MIN_P
#define IGS_FWD_WAVE_MIN_P 8
#endif
__host__ __device__ constexpr bool fwd_wave_lists(int C) { return fwd_sep_p(C) >= IGS_FWD_WAVE_MIN_P; }

// A tile's list is cut into S parts for S workgroups (blockIdx.y). The parts shrink linearly from
// (1 + ramp) to (1 - ramp) times the mean: workgroups start part by part, so the last to start are
// the shortest (B=16 N=8192 256x256: forward 1.30 ms with equal parts, 1.23 ms with ramp 0.6 to 0.8).
// Where the whole launch is resident at once (small problems) nothing starts later, the longest part
// decides, and the parts are equal (B=1 N=2048 256x256: fit step 146 -> 141 us).
#ifndef IGS_SPLIT_RAMP
#define IGS_SPLIT_RAMP 0.7f
#endif
constexpr float kSplitRamp = IGS_SPLIT_RAMP;

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
    if (rec_has_yrange(C)) {
        g.ylo = v[6 + C];
        g.yhi = v[7 + C];
    } else {
        g.ylo = g.yhi = 0.0f;
    }
    return g;
}

// A forward record of the separable kernels (sep_terms): px, py, sD, skD, A'' (q' = -(sD dy + skD dx)^2 +
// A'' dx^2), alpha, alpha*c_0.., the tag (sD again, or NaN where the form has no completed square) and
// A', B2', D' for the evaluation term by term.  The completed square needs the first 7 + C floats only.
template <int C>
struct FRec {
    float px, py, sD, skD, A2, al;
    float ac[C];
    float tag;
};
template <int C>
__device__ __forceinline__ FRec<C> lds_frec(const float4* r) {
    constexpr int R4 = (7 + C + 3) / 4;
    float v[4 * R4];
#pragma unroll
    for (int i = 0; i < R4; ++i) {
        const float4 t = r[i];
        v[4 * i] = t.x;
        v[4 * i + 1] = t.y;
        v[4 * i + 2] = t.z;
        v[4 * i + 3] = t.w;
    }
    FRec<C> g;
    g.px = v[0];
    g.py = v[1];
    g.sD = v[2];
    g.skD = v[3];
    g.A2 = v[4];
    g.al = v[5];
#pragma unroll
    for (int c = 0; c < C; ++c) g.ac[c] = v[6 + c];
    g.tag = v[6 + C];
    return g;
}
// A', B2', D' of a forward record (floats 7 + C .. 9 + C)
template <int C>
__device__ __forceinline__ void lds_frec_terms(const float4* r, float& A, float& B2, float& D) {
    const float* f = reinterpret_cast<const float*>(r);
    A = f[7 + C];
    B2 = f[8 + C];
    D = f[9 + C];
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
// workgroup through the double-buffered LDS window sh[2][CH*R4]; body(rec, lds) runs once per record
// with its first RD float4 in registers (read from a wave-uniform LDS address) and the wave-uniform
// LDS pointer to the whole record.  Records past `count` in the last chunk
// read as all-zero (for a Gaussian record: alpha = 0, adds exactly 0).  Must be called by all
// NT threads of the workgroup (it contains barriers; with NT = 64, one wave, they cost nothing).
// With kGather, record i of the stream is src record index[i] (a tile's Gaussian list).
// The general form: fetch(lds record) returns the registers one evaluation reads, body(those, lds record) is
// the evaluation; kGrouped: body(the registers of the kStreamUnroll records of a group, lds record of the
// first) runs once per group.
template <int R4, int CH, bool kGather, int NT, bool kGrouped, class Fetch, class Body>
__device__ __forceinline__ void stream_records_lds_f(const float4* __restrict__ src, int count,
                                                     float4* sh, Fetch&& fetch, Body&& body,
                                                     const int* __restrict__ index) {
    constexpr int E = CH * R4;                          // float4 per chunk
    constexpr int PRE = (E + NT - 1) / NT;              // float4 per thread per chunk
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
            const int e = i * NT + tid, ge = chunk * E + e;
            idx[i] = (kGather && e < E && ge < total) ? index[ge / R4] : 0;
        }
    };
    float4 pre[PRE];
    auto load_records = [&](int chunk) {
#pragma unroll
        for (int i = 0; i < PRE; ++i) {
            const int e = i * NT + tid, ge = chunk * E + e;
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
        const int e = i * NT + tid;
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
        // (the last chunk stops after its last record's group; the slots behind it hold zeros)
        const int lim = min(CH, (count - k * CH + kStreamUnroll - 1) / kStreamUnroll * kStreamUnroll);
#pragma unroll 1
        for (int n = 0; n < lim; n += kStreamUnroll) {
            decltype(fetch(cur)) rr[kStreamUnroll];
#pragma unroll
            for (int u = 0; u < kStreamUnroll; ++u) rr[u] = fetch(cur + (n + u) * R4);
            __builtin_amdgcn_sched_barrier(0);
            if constexpr (kGrouped) {
                body(rr, cur + n * R4);
                __builtin_amdgcn_sched_barrier(0);
            } else {
#pragma unroll
                for (int u = 0; u < kStreamUnroll; ++u) {
                    body(rr[u], cur + (n + u) * R4);
                    __builtin_amdgcn_sched_barrier(0);
                }
            }
        }
        if (k + 1 < chunks) {
            float4* nxt = sh + ((k + 1) & 1) * E;
#pragma unroll
            for (int i = 0; i < PRE; ++i) {
                const int e = i * NT + tid;
                if (e < E) nxt[e] = pre[i];
            }
        }
        __syncthreads();
    }
}

// The first RD float4 of a record as the registers of an evaluation.
template <int RD>
struct RecHead {
    float4 v[RD];
};
template <int RD>
__device__ __forceinline__ RecHead<RD> rec_head(const float4* rec) {
    RecHead<RD> h;
#pragma unroll
    for (int i = 0; i < RD; ++i) h.v[i] = rec[i];
    return h;
}
template <int R4, int CH, bool kGather = false, int NT = kThreads, int RD = R4, class Body>
__device__ __forceinline__ void stream_records_lds(const float4* __restrict__ src, int count,
                                                   float4* sh, Body&& body,
                                                   const int* __restrict__ index = nullptr) {
    stream_records_lds_f<R4, CH, kGather, NT, false>(
        src, count, sh, [](const float4* rec) { return rec_head<RD>(rec); },
        [&](const RecHead<RD>& h, const float4* lds) { body(h.v, lds); }, index);
}

// The same stream for one wave on its own (wave-uniform `count`, `index` and buffers; no barrier, so
// the waves of a workgroup may run it with different lists), without staging registers: the records of the next
// chunk go from global memory straight into the other LDS buffer (global_load_lds_dwordx4: lane l
// of the instruction writes 16 bytes at base + 16 l) while the current one is computed, and one
// vmcnt wait per chunk separates the two.  Slots past `count` load the all-zero record `zero_rec`.
// The two buffers are separate arrays and the chunk loop is unrolled by two, so that every LDS read
// names the buffer it reads.
// (fetch, body and kGrouped as in stream_records_lds_f)
template <int R4, int CH, bool kGrouped, class Fetch, class Body>
__device__ __forceinline__ void stream_records_dma_f(const float4* __restrict__ src,
                                                     const float4* __restrict__ zero_rec, int count,
                                                     float4* sh0, float4* sh1, Fetch&& fetch, Body&& body,
                                                     const int* __restrict__ index) {
    constexpr int E = CH * R4;  // float4 per chunk
    static_assert(E % 64 == 0 && CH % kStreamUnroll == 0, "a chunk is a whole number of wave loads");
    constexpr int PRE = E / 64;
    const int lane = threadIdx.x & 63;
    const int total = count * R4;
    const int chunks = (count + CH - 1) / CH;
    int idx[PRE];
    auto load_idx = [&](int chunk) {
#pragma unroll
        for (int i = 0; i < PRE; ++i) {
            const int ge = chunk * E + i * 64 + lane;
            idx[i] = ge < total ? index[ge / R4] : -1;
        }
    };
    auto issue = [&](float4* buf) {  // the records whose indices load_idx fetched last
#pragma unroll
        for (int i = 0; i < PRE; ++i) {
            const int part = (i * 64 + lane) % R4;  // E % R4 == 0: the same in every chunk
            const float4* p = idx[i] >= 0 ? src + (size_t)idx[i] * R4 + part : zero_rec + part;
            // Written as assembly: the compiler's wait-count pass, which follows the builtin form of
            // this load, puts a vmcnt(0) in front of the LDS reads of whichever buffer sits at LDS
            // address 0 (it no longer knows which array such a read belongs to), and the loads into
            // the other buffer would not overlap with the compute.  The waits are `landed` below.
            const unsigned lds = __builtin_amdgcn_readfirstlane(
                (unsigned)(__UINTPTR_TYPE__)(__attribute__((address_space(3))) float4*)(buf + i * 64));
            unsigned m0_saved;  // M0 is put back: the compiler does not honour a clobber of it
            asm volatile("s_mov_b32 %0, m0\n\ts_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off\n\t"
                         "s_nop 0\n\ts_mov_b32 m0, %0"
                         : "=&s"(m0_saved)
                         : "v"(p), "s"(lds)
                         : "memory");
        }
    };
    auto landed = [] { asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); };
    auto compute = [&](const float4* cur, int k) {
        // (the last chunk stops after its last record's group; the slots behind it hold zeros)
        const int lim = min(CH, (count - k * CH + kStreamUnroll - 1) / kStreamUnroll * kStreamUnroll);
#pragma unroll 1
        for (int n = 0; n < lim; n += kStreamUnroll) {
            decltype(fetch(cur)) rr[kStreamUnroll];
#pragma unroll
            for (int u = 0; u < kStreamUnroll; ++u) rr[u] = fetch(cur + (n + u) * R4);
            __builtin_amdgcn_sched_barrier(0);
            if constexpr (kGrouped) {
                body(rr, cur + n * R4);
                __builtin_amdgcn_sched_barrier(0);
            } else {
#pragma unroll
                for (int u = 0; u < kStreamUnroll; ++u) {
                    body(rr[u], cur + (n + u) * R4);
                    __builtin_amdgcn_sched_barrier(0);
                }
            }
        }
    };
    if (chunks == 0) return;
    load_idx(0);
    issue(sh0);
    load_idx(1);
    landed();
    for (int k = 0; k < chunks; k += 2) {
        if (k + 1 < chunks) {
            issue(sh1);
            load_idx(k + 2);
        }
        compute(sh0, k);
        landed();
        if (k + 1 >= chunks) break;
        if (k + 2 < chunks) {
            issue(sh0);
            load_idx(k + 3);
        }
        compute(sh1, k + 1);
        landed();
    }
}

template <int R4, int CH, int RD = R4, class Body>
__device__ __forceinline__ void stream_records_dma(const float4* __restrict__ src,
                                                   const float4* __restrict__ zero_rec, int count,
                                                   float4* sh0, float4* sh1, Body&& body,
                                                   const int* __restrict__ index) {
    stream_records_dma_f<R4, CH, false>(
        src, zero_rec, count, sh0, sh1, [](const float4* rec) { return rec_head<RD>(rec); },
        [&](const RecHead<RD>& h, const float4* lds) { body(h.v, lds); }, index);
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

// Separable grid: lane = one column, P consecutive rows; wave = 64 columns x P rows (kWave = false) or
// kWaveCols columns x 64 / kWaveCols blocks of P rows (kWave = true).  The square is completed along
// the column (sep_terms): q' = -(sD dy + skD dx)^2 + A'' dx^2 = -u^2 + c0 with
// u = sD y' + (skD dx - sD py'), y' and py' relative to the lane's middle row so that the hoisted term
// carries no more rounding than u itself.  Per Gaussian and lane: dx, A''dx^2, py', the hoisted term of u
// once (6 instructions), then per pixel 2 fma, exp2, 1 + C fma.  Records without a completed square, or
// with sD times the largest |y'| of the wave above kSepSpanLimitFwd (one wave-uniform comparison of the tag
// with the wave's limit), are evaluated term by term: q' = (D' dy + B2' dx) dy + A' dx^2.
// kWave = false: workgroup = wx x (4/wx) waves, all four streaming the tile's Gaussian list.
// kWave = true (fwd_wave_lists): every wave has a list of its own and streams it independently of
// the others (no barrier in the kernel); the four waves of a workgroup are the rectangles of one
// 64 x 4P tile of the binning.
// (kOne: launched as workgroups of one wave; only with kWave)
#ifndef IGS_FWD_MIN_WAVES
#define IGS_FWD_MIN_WAVES 3
#endif
// The accumulation out[pixel][channel] += w[pixel] (alpha, alpha c_0, ..)[channel] over the Gaussians is a
// rank-1 update of a 64 x (1 + C) matrix per row of pixels.  v_mfma_f32_4x4x1_16b_f32 (16 blocks of 4 x 4,
// K = 1) with A = four channel values (lane 4 b + i holds channel i, the same in all blocks) and B = the row's
// weights (lane = pixel) leaves channel i of pixel `lane` in register i of the lane: the layout of the vector
// form, full fp32, the same order of summation, one matrix instruction of two passes for four vector FMAs.
// The matrix instructions of a group of records are issued back to back behind the group's vector
// arithmetic: a vector instruction behind a matrix one waits for it to drain, and alternating the two was
// slower than no matrix instructions at all (B=16 N=8192 256x256 C=3 forward call: vector 0.972 ms, matrix in
// phases 0.876, alternating 1.03-1.13).
// Where a row's last matrix instruction would be mostly padding the vector form stays: one channel (2 of 4 used:
// B=4 N=8192 256x256 forward 0.251 -> 0.268 ms) and four (5 of 8: 0.343 -> 0.340); with 2, 3, 8, 12 and 16
// channels the same shape gains 1.5, 9, 2.5, 6 and 3 %.
#ifndef IGS_FWD_MFMA
#define IGS_FWD_MFMA 1
#endif
__host__ __device__ constexpr bool fwd_mfma(int C) { return IGS_FWD_MFMA && C != 1 && C != 4; }
typedef float fwd_v4f __attribute__((ext_vector_type(4)));
template <int C, int P, bool kWave, bool kOne = false>
__global__ __launch_bounds__(kThreads, P >= 16 ? IGS_FWD_MIN_WAVES : 1) void k_fwd_sep(const FwdArgs a) {  // (16 rows per lane: three waves per SIMD, i.e. at most 168 registers)
    static_assert(kWave || !kOne, "one-wave workgroups need a list per wave");
    constexpr bool kSq = fwd_square(C);  // completed square (its own records) or term by term (the plain ones)
    static_assert(kSq == (P >= 8) || !IGS_FWD_SQUARE, "the completed square goes with 8 or more rows per lane");
    constexpr int RS = kSq ? frec_stride_of(C) : rec_stride_of(C), R4 = RS / 4;
    constexpr int RD = kSq ? (7 + C + 3) / 4 : R4;  // float4 of a record that every evaluation reads
    constexpr bool kMfma = fwd_mfma(C);  // the sums on the matrix cores
    constexpr int NM = (C + 4) / 4;      // matrix instructions per row of pixels: four of the 1 + C channels each
    static_assert(!kMfma || kSq == kWave, "matrix form: completed-square records with a list per wave, or plain ones with a shared list");
    IGS_GATE(a);
    // Waves with lists of their own can be launched as workgroups of one wave (kOne): the four
    // waves of a tile share nothing, and a wave slot then frees as soon as its wave ends instead
    // of when the longest list of the four does.  Workgroup q: XCD q % 8, there tile (q / 8) / 4
    // of the XCD's range and wave rectangle (q / 8) % 4 of that tile.
    const int q = kOne ? (int)(blockIdx.x & 7) + 8 * (int)(blockIdx.x >> 5) : (int)blockIdx.x;
    // (each part of the lists starts one tile further on in the XCD's range: the workgroups of consecutive parts
    // otherwise reach the compute units in the same tile order, and where a few tiles hold most of the work --
    // Gaussians crowded around the image centre -- the same units get the long lists every time: B=8 N=4096
    // 256x256 at a module's initialisation, forward kernel 89 -> 82 us; 3, 5 or 7 tiles: 84-88)
    // A single image: every XCD reads all of its Gaussians anyway, and a contiguous range of tiles would give
    // the XCDs that hold the top and the bottom rows the short lists (B=1 N=16384 512x512: 43 000-67 000 list
    // entries per XCD).  The tiles are dealt round-robin instead, each tile row shifted against the one above so
    // that an XCD does not end up with one tile column: forward call 0.207 -> 0.199 ms.
    const bool dealt = a.B == 1;
    const int tile = dealt ? q : xcd_contiguous_from(q, a.total_tiles, (int)blockIdx.y);
    if (tile >= a.total_tiles) return;  // workgroup-uniform
    const int per_img = a.tiles_x * a.tiles_y;
    const int b = tile / per_img;
    const int tl = tile - b * per_img;
    const int ty = tl / a.tiles_x;
    const int tx = dealt ? (tl - ty * a.tiles_x + 3 * ty + (int)blockIdx.y) % a.tiles_x : tl - ty * a.tiles_x;
    const int wave = kOne ? (int)((blockIdx.x >> 3) & 3) : (int)(threadIdx.x >> 6);
    const int lane = threadIdx.x & 63;
    // A wave with a list of its own covers kWaveCols columns x (64 / kWaveCols) P rows: lane l has
    // column l % kWaveCols and the P rows of row block l / kWaveCols; the tile of four waves is 64
    // columns x 4 P rows either way.
    // With a shared list (kWave = false) the workgroup is wx waves of wcols columns side by side, 4 / wx
    // down: 64 wx columns x (4 / wx) P rows, or 32 columns x 8 P rows.
    constexpr int kHalves = 64 / kWaveCols;
    const int wx = kWave ? kHalves : a.wx;
    const int wcols = kWave ? kWaveCols : a.wcols;
    const int wxi = wave % wx, wyi = wave / wx;
    const int col = (tx * wx + wxi) * wcols + lane % wcols;
    const int row0 = ((ty * (4 / wx) + wyi) * (64 / wcols) + lane / wcols) * P;
    const float xv = a.x[b * a.sxb + (long)min(col, a.W - 1) * a.sxw];
    float yv[P];
    // (all P loads first, then the pins: a pin right behind its load would wait for each load in turn)
#pragma unroll
    for (int p = 0; p < P; ++p) yv[p] = a.y[b * a.syb + (long)min(row0 + p, a.H - 1) * a.syh];
#pragma unroll
    for (int p = 0; p < P; ++p) yv[p] = in_vgpr(yv[p]);

    float dsum[P], num[P][C];
    [[maybe_unused]] fwd_v4f acc[kMfma ? P : 1][NM];  // matrix form: channel 4 m + i of row p in acc[p][m][i]
#pragma unroll
    for (int p = 0; p < P; ++p) {
        dsum[p] = 0.0f;
#pragma unroll
        for (int c = 0; c < C; ++c) num[p][c] = 0.0f;
    }
#pragma unroll
    for (int p = 0; p < (kMfma ? P : 1); ++p)
#pragma unroll
        for (int m = 0; m < NM; ++m) acc[p][m] = fwd_v4f{0.0f, 0.0f, 0.0f, 0.0f};
    float wylo = yv[0], wyhi = yv[0];  // y range of this wave's rows (NaN-safe: see the test below)
    bool ybad = !(yv[0] == yv[0]);
#pragma unroll
    for (int p = 1; p < P; ++p) {
        wylo = fminf(wylo, yv[p]);
        wyhi = fmaxf(wyhi, yv[p]);
        ybad = ybad || !(yv[p] == yv[p]);
    }
    if (ybad) {
        wylo = -__builtin_inff();
        wyhi = __builtin_inff();
    }
    // With the completed square the rows are, from here on, relative to the lane's middle row yc, if that
    // loses nothing (yv - yc is exact for the neighbouring rows of an ordinary grid; where coordinates
    // jump within a wave's rows it is not, and the wave keeps them as they are, yc = 0).
    float yc = 0.0f, span = 0.0f;
    if (kSq) {
        const float mid = yv[P / 2];
        bool exact = true;
#pragma unroll
        for (int p = 0; p < P; ++p) exact = exact && ((yv[p] - mid) + mid == yv[p]);
        yc = __ballot(!exact) == 0ull ? mid : 0.0f;
#pragma unroll
        for (int p = 0; p < P; ++p) {
            yv[p] = in_vgpr(yv[p] - yc);
            span = fmaxf(span, fabsf(yv[p]));
        }
        if (ybad) span = __builtin_nanf("");
        if (wcols == 32) {  // two row blocks per wave: the larger of the two (NaN if either is)
            const float o = __shfl_xor(span, 32);
            span = (span != span || o != o) ? __builtin_nanf("") : fmaxf(span, o);
        }
    }
    // records with tag = sD <= sd_limit take the completed square (a NaN on either side: term by term)
    const float sd_limit = in_vgpr(fminf(kSepSpanLimitFwd / span, 3.0e38f));
    // this unit's Gaussians (those whose ellipse reaches it), split S ways by list position
    const int s = blockIdx.y;
    // (wave lists are numbered by rectangle, row after row; rectangles outside the image have none)
    const int rrow = ty * (4 / kHalves) + wyi, rcol = tx * kHalves + wxi;
    const size_t li = (size_t)b * a.list_img + (size_t)(kWave ? rrow : ty) * a.list_row + (kWave ? rcol : tx);
    const int count = (!kWave || (rrow * kHalves * P < a.H && rcol * kWaveCols < a.W)) ? a.counts[li] : 0;
    // parts of decreasing length: part i has weight 1 + ramp - 2 ramp i / (S - 1), the sum is S
    auto cut = [&](int i) {  // first entry of part i, a multiple of 4
        const float f = a.S > 1 ? (float)i * (1.0f + a.ramp - a.ramp * (float)(i - 1) / (float)(a.S - 1)) / (float)a.S
                                : (float)i;
        return min(count, ((int)((float)count * f) + 3) & ~3);
    };
    const int n0 = cut(s);
    const int n1 = s + 1 == a.S ? count : cut(s + 1);
    const int* list = a.lists + li * a.Np + n0;
    const float4* src = reinterpret_cast<const float4*>((kSq ? a.frecs : a.packed) + (size_t)b * a.Np * RS);
    // the exponents of the lane's P pixels for one record, and its alpha and alpha*c
    // completed-square records (px, py, sD, skD, A'', tag of `g`; `terms`: where the record's A', B2', D' are read from)
    auto sq_exponents = [&](const FRec<C>& g, const float4* terms, float (&e)[P]) {
            const float dx = xv - g.px;
            const float pyl = g.py - yc;
            if (__ballot(g.tag <= sd_limit) != 0ull) {  // wave-uniform: both sides are
                const float c0 = (g.A2 * dx) * dx;
                const float off = fmaf(g.skD, dx, -(g.sD * pyl));
#pragma unroll
                for (int p = 0; p < P; ++p) {
                    const float u = fmaf(g.sD, yv[p], off);
                    e[p] = fmaf(-u, u, c0);
                }
            } else {  // no completed square, or its scale is too large for this wave's rows
                float Ap, B2p, Dp;
                lds_frec_terms<C>(terms, Ap, B2p, Dp);
                // py - yc = pyl + lo exactly (two-sum), so that dy = y - py carries one rounding, as without
                // the shift (the sharp Gaussians that come here need it); lo, half an ulp of pyl at most,
                // goes into the constant and the linear coefficient of the form in dy0 = y' - pyl:
                // q' = (D' dy0 + c1 - 2 D' lo) dy0 + (c0 - c1 lo), up to D' lo^2 < 1e-9
                const float bb = pyl - g.py;
                const float lo = (g.py - (pyl - bb)) + (-yc - bb);
                const float c1p = B2p * dx;
                const float c0 = fmaf(-c1p, lo, (Ap * dx) * dx);
                const float c1 = fmaf(-2.0f * Dp, lo, c1p);
#pragma unroll
                for (int p = 0; p < P; ++p) {
                    const float dy = yv[p] - pyl;
                    const float t = fmaf(Dp, dy, c1);
                    e[p] = fmaf(t, dy, c0);
                }
            }
    };
    // plain records, term by term (px, py, A', B2', D' of `g`)
    auto plain_exponents = [&](const GRec<C>& g, float (&e)[P]) {
        const float dx = xv - g.px;
        const float adx = g.A * dx;
        const float c0 = adx * dx;
        const float c1 = g.B2 * dx;
#pragma unroll
        for (int p = 0; p < P; ++p) {
            const float dy = yv[p] - g.py;
            const float t = fmaf(g.D, dy, c1);
            e[p] = fmaf(t, dy, c0);
        }
    };
    auto exponents = [&](auto wave_skip, const float4* r, const float4* lds, float (&e)[P], float& al, float (&ac)[C]) -> bool {
        if constexpr (kSq) {
            const FRec<C> g = lds_frec<C>(r);
            al = g.al;
#pragma unroll
            for (int c = 0; c < C; ++c) ac[c] = g.ac[c];
            sq_exponents(g, RD == R4 ? r : lds, e);
        } else {
            const GRec<C> g = lds_grec<C>(r);
            // A list shared by four waves of P rows each: a wave whose own rows the reach box misses
            // skips the record (wave-uniform: the record is the same in all lanes).
            if (decltype(wave_skip)::value && __ballot(!(g.yhi < wylo || g.ylo > wyhi)) == 0ull) return false;
            al = g.al;
#pragma unroll
            for (int c = 0; c < C; ++c) ac[c] = g.ac[c];
            plain_exponents(g, e);
        }
        return true;
    };
    auto body = [&](auto wave_skip, const float4* r, const float4* lds) {
        // three phases, so that the P independent chains overlap their latencies and the
        // transcendental ops issue back to back
        float e[P], al, ac[C];
        if (!exponents(wave_skip, r, lds, e, al, ac)) return;
#pragma unroll
        for (int p = 0; p < P; ++p) e[p] = hw_exp2(e[p]);
#pragma unroll
        for (int p = 0; p < P; ++p) {
            dsum[p] = fmaf(e[p], al, dsum[p]);
#pragma unroll
            for (int c = 0; c < C; ++c) num[p][c] = fmaf(e[p], ac[c], num[p][c]);
        }
    };
    // The per-wave test of a shared list costs a few percent when it never fires, so it is used only
    // for tiles that fewer than 7/8 of the Gaussians reach (workgroup-uniform choice of the loop):
    // there some boxes are small against the image, and those are often small against the tile too.
    // Matrix form: per record one float4 and the few floats behind it that the exponents need, and per matrix
    // instruction one float read at a lane-dependent address: channel min(4 m + lane % 4, C) of the record
    // (channel 0 = alpha, 1 + c = alpha c_c: floats 5.. of both record layouts).  A group's exponentials
    // first, then its matrix instructions.
    [[maybe_unused]] const int chl = lane & 3;
    [[maybe_unused]] auto channel_values = [&](const float4* rec, float (&cv)[NM]) {
        const float* f = reinterpret_cast<const float*>(rec);
#pragma unroll
        for (int m = 0; m < NM; ++m) cv[m] = f[5 + min(4 * m + chl, C)];
    };
    [[maybe_unused]] auto accumulate = [&](const float (&cv)[NM], const float (&e)[P]) {
#pragma unroll
        for (int p = 0; p < P; ++p)
#pragma unroll
            for (int m = 0; m < NM; ++m) acc[p][m] = __builtin_amdgcn_mfma_f32_4x4x1f32(cv[m], e[p], acc[p][m], 0, 0, 0);
    };
    if constexpr (kMfma && kWave) {
        __shared__ float4 sh0[kOne ? 1 : 4][kGaussChunk * R4];  // per wave: the two chunk buffers
        __shared__ float4 sh1[kOne ? 1 : 4][kGaussChunk * R4];
        struct Head {
            float4 r0;  // px, py, sD, skD
            float a2, tag, cv[NM];
        };
        stream_records_dma_f<R4, kGaussChunk, true>(
            src, reinterpret_cast<const float4*>(a.zero_rec), n1 - n0, sh0[kOne ? 0 : wave], sh1[kOne ? 0 : wave],
            [&](const float4* rec) {
                const float* f = reinterpret_cast<const float*>(rec);
                Head h;
                h.r0 = rec[0];
                h.a2 = f[4];
                h.tag = f[6 + C];
                channel_values(rec, h.cv);
                return h;
            },
            [&](const Head (&h)[kStreamUnroll], const float4* lds) {
                float e[kStreamUnroll][P];
#pragma unroll
                for (int u = 0; u < kStreamUnroll; ++u) {
                    FRec<C> g;
                    g.px = h[u].r0.x;
                    g.py = h[u].r0.y;
                    g.sD = h[u].r0.z;
                    g.skD = h[u].r0.w;
                    g.A2 = h[u].a2;
                    g.tag = h[u].tag;
                    sq_exponents(g, lds + u * R4, e[u]);
                }
#pragma unroll
                for (int u = 0; u < kStreamUnroll; ++u)
#pragma unroll
                    for (int p = 0; p < P; ++p) e[u][p] = hw_exp2(e[u][p]);
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int u = 0; u < kStreamUnroll; ++u) accumulate(h[u].cv, e[u]);
            },
            list);
    } else if constexpr (kMfma) {
        __shared__ float4 sh[2 * kGaussChunk * R4];
        struct Head {
            float4 r0;  // px, py, A', B2'
            float D, ylo, yhi, cv[NM];
        };
        auto head = [&](const float4* rec) {
            const float* f = reinterpret_cast<const float*>(rec);
            Head h;
            h.r0 = rec[0];
            h.D = f[4];
            h.ylo = rec_has_yrange(C) ? f[6 + C] : 0.0f;
            h.yhi = rec_has_yrange(C) ? f[7 + C] : 0.0f;
            channel_values(rec, h.cv);
            return h;
        };
        auto group = [&](auto wave_skip, const Head (&h)[kStreamUnroll]) {
            float e[kStreamUnroll][P];
            bool reached[kStreamUnroll];  // wave-uniform: the record's reach box meets this wave's rows
#pragma unroll
            for (int u = 0; u < kStreamUnroll; ++u) {
                reached[u] = !(decltype(wave_skip)::value && __ballot(!(h[u].yhi < wylo || h[u].ylo > wyhi)) == 0ull);
                if (reached[u]) {
                    GRec<C> g;
                    g.px = h[u].r0.x;
                    g.py = h[u].r0.y;
                    g.A = h[u].r0.z;
                    g.B2 = h[u].r0.w;
                    g.D = h[u].D;
                    plain_exponents(g, e[u]);
#pragma unroll
                    for (int p = 0; p < P; ++p) e[u][p] = hw_exp2(e[u][p]);
                }
            }
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int u = 0; u < kStreamUnroll; ++u)
                if (reached[u]) accumulate(h[u].cv, e[u]);
        };
        // (the per-wave test of a shared list: see below)
        if (rec_has_yrange(C) && 8L * count < 7L * a.Np)
            stream_records_lds_f<R4, kGaussChunk, true, kThreads, true>(
                src, n1 - n0, sh, head, [&](const Head (&h)[kStreamUnroll], const float4*) { group(std::true_type{}, h); }, list);
        else
            stream_records_lds_f<R4, kGaussChunk, true, kThreads, true>(
                src, n1 - n0, sh, head, [&](const Head (&h)[kStreamUnroll], const float4*) { group(std::false_type{}, h); }, list);
    } else if constexpr (kWave) {
        __shared__ float4 sh0[kOne ? 1 : 4][kGaussChunk * R4];  // per wave: the two chunk buffers
        __shared__ float4 sh1[kOne ? 1 : 4][kGaussChunk * R4];
        stream_records_dma<R4, kGaussChunk, RD>(
            src, reinterpret_cast<const float4*>(a.zero_rec), n1 - n0, sh0[kOne ? 0 : wave], sh1[kOne ? 0 : wave],
            [&](const float4* r, const float4* lds) { body(std::false_type{}, r, lds); }, list);
    } else {
        __shared__ float4 sh[2 * kGaussChunk * R4];
        if (!kSq && rec_has_yrange(C) && 8L * count < 7L * a.Np)
            stream_records_lds<R4, kGaussChunk, true, kThreads, RD>(
                src, n1 - n0, sh, [&](const float4* r, const float4* lds) { body(std::true_type{}, r, lds); }, list);
        else
            stream_records_lds<R4, kGaussChunk, true, kThreads, RD>(
                src, n1 - n0, sh, [&](const float4* r, const float4* lds) { body(std::false_type{}, r, lds); }, list);
    }
    if constexpr (kMfma) {
#pragma unroll
        for (int p = 0; p < P; ++p) {
            dsum[p] = acc[p][0][0];
#pragma unroll
            for (int c = 0; c < C; ++c) num[p][c] = acc[p][(1 + c) / 4][(1 + c) % 4];
        }
    }
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
    // the weights of the lane's P pixels for a record (px, py, A', B2' in r0)
    auto weights = [&](const float4& r0, float D, float (&e)[P]) {
#pragma unroll
        for (int j = 0; j < P; ++j) {
            const float dx = xv[j] - r0.x;
            const float dy = yv[j] - r0.y;
            float t = r0.z * dx;
            t = fmaf(r0.w, dy, t);
            const float v = D * dy;
            float q = t * dx;
            e[j] = fmaf(v, dy, q);
        }
#pragma unroll
        for (int j = 0; j < P; ++j) e[j] = hw_exp2(e[j]);
    };
    if constexpr (fwd_mfma(C)) {
        // the sums as matrix instructions, a group's behind its vector arithmetic (see k_fwd_sep)
        constexpr int NM = (C + 4) / 4;
        fwd_v4f acc[P][NM];
#pragma unroll
        for (int j = 0; j < P; ++j)
#pragma unroll
            for (int m = 0; m < NM; ++m) acc[j][m] = fwd_v4f{0.0f, 0.0f, 0.0f, 0.0f};
        const int chl = threadIdx.x & 3;
        struct Head {
            float4 r0;
            float D, cv[NM];
        };
        stream_records_lds_f<R4, kGaussChunk, false, kThreads, true>(
            src, n1 - n0, sh,
            [&](const float4* rec) {
                const float* f = reinterpret_cast<const float*>(rec);
                Head h;
                h.r0 = rec[0];
                h.D = f[4];
#pragma unroll
                for (int m = 0; m < NM; ++m) h.cv[m] = f[5 + min(4 * m + chl, C)];
                return h;
            },
            [&](const Head (&h)[kStreamUnroll], const float4*) {
                float e[kStreamUnroll][P];
#pragma unroll
                for (int u = 0; u < kStreamUnroll; ++u) weights(h[u].r0, h[u].D, e[u]);
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int u = 0; u < kStreamUnroll; ++u)
#pragma unroll
                    for (int j = 0; j < P; ++j)
#pragma unroll
                        for (int m = 0; m < NM; ++m)
                            acc[j][m] = __builtin_amdgcn_mfma_f32_4x4x1f32(h[u].cv[m], e[u][j], acc[j][m], 0, 0, 0);
            },
            nullptr);
#pragma unroll
        for (int j = 0; j < P; ++j) {
            dsum[j] = acc[j][0][0];
#pragma unroll
            for (int c = 0; c < C; ++c) num[j][c] = acc[j][(1 + c) / 4][(1 + c) % 4];
        }
    } else {
        stream_records_lds<R4, kGaussChunk>(src, n1 - n0, sh, [&](const float4* r, const float4*) {
            const GRec<C> g = lds_grec<C>(r);
            float e[P];
            weights(r[0], g.D, e);
#pragma unroll
            for (int j = 0; j < P; ++j) {
                dsum[j] = fmaf(e[j], g.al, dsum[j]);
#pragma unroll
                for (int c = 0; c < C; ++c) num[j][c] = fmaf(e[j], g.ac[c], num[j][c]);
            }
        });
    }
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
    // 64 pixels x 4 channel lanes per workgroup: lane k sums channels k, k+4, ... (channel C is
    // the denominator), the partials of 8 splits are loaded together; the pixel's denominator
    // reaches the other lanes through LDS.
    constexpr int kPix = 64, kLanes = kThreads / kPix, kBatch = 8;
    __shared__ float dsh[kPix];
    if (flag != nullptr && *flag != want) return;
    const int pl = threadIdx.x % kPix, k = threadIdx.x / kPix;
    const int p = blockIdx.x * kPix + pl;
    const int b = blockIdx.y;
    const bool valid = p < HW;
    const int pc = min(p, HW - 1);
    auto sum_channel = [&](int c) -> float {
        const float* src = part + ((size_t)b * (C + 1) + c) * HW + pc;
        const size_t stride = (size_t)B * (C + 1) * HW;
        float v = 0.0f;
        for (int s0 = 0; s0 < S; s0 += kBatch) {
            float t[kBatch];
#pragma unroll
            for (int j = 0; j < kBatch; ++j) t[j] = s0 + j < S ? src[(size_t)(s0 + j) * stride] : 0.0f;
#pragma unroll
            for (int j = 0; j < kBatch; ++j) v += t[j];  // fixed order s = 0, 1, ...
        }
        return v;
    };
    constexpr int kMine = (IGS_MAX_CHANNELS + 1 + kLanes - 1) / kLanes;
    float mine[kMine];
#pragma unroll
    for (int j = 0; j < kMine; ++j) {
        const int c = k + j * kLanes;
        mine[j] = 0.0f;
        if (c <= C) {
            mine[j] = sum_channel(c);
            if (c == C) dsh[pl] = mine[j];
        }
    }
    __syncthreads();
    const float d = dsh[pl];
    const float inv = 1.0f / (d + eps);
#pragma unroll
    for (int j = 0; j < kMine; ++j) {
        const int c = k + j * kLanes;
        if (!valid || c > C) continue;
        if (c == C)
            den[(size_t)b * HW + p] = d;
        else
            out[((size_t)b * C + c) * HW + p] = mine[j] * inv;
    }
}
