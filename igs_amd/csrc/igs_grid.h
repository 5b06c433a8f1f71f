// igs_grid.h -- gradients w.r.t. the grids and the device-side grid classification.
// Included by igs_gs2d.hip inside its anonymous namespace (one translation unit).
#pragma once

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
    const int* flag;  // AUTO grid mode: run only if *flag == want
    int want;
};

template <int C, int P>
__global__ __launch_bounds__(kThreads) void k_bwd_grid(const GridGradArgs a) {
    constexpr int RS = rec_stride_of(C), R4 = RS / 4;
    __shared__ float4 sh[2 * kGaussChunk * R4];
    IGS_GATE(a);
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
    stream_records_lds<R4, kGaussChunk>(src, a.Np, sh, [&](const float4* r, const float4*) {
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

// Grid gradients of the general backward with the grid sums fused in (k_bwd_gen_grid): adds
// the `groups` workgroup partials of every pixel in order and applies the factor -1/k.
__global__ __launch_bounds__(kThreads) void k_grid_reduce(const float2* __restrict__ part, int groups, int HW,
                                                          int HWp, float* __restrict__ gx, float* __restrict__ gy,
                                                          const int* __restrict__ flag, int want) {
    if (flag != nullptr && *flag != want) return;
    const int p = blockIdx.x * kThreads + threadIdx.x;
    const int b = blockIdx.y;
    if (p >= HW) return;
    float sx = 0.0f, sy = 0.0f;
    for (int g = 0; g < groups; ++g) {
        const float2 v = part[((size_t)b * groups + g) * HWp + p];
        sx += v.x;
        sy += v.y;
    }
    constexpr float kScale = -1.0f / kNegHalfLog2e;
    gx[(size_t)b * HW + p] = kScale * sx;
    gy[(size_t)b * HW + p] = kScale * sy;
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
