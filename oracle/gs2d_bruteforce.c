/* Scalar fp64 brute force of the 2-D Gaussian splat and its analytic gradients.
 *
 * TEST INFRASTRUCTURE ONLY: an independent pin for oracle/gs2d_oracle.py, written in a
 * different language with plain loops.  Never linked into or called from the product.
 *
 * Forward restates naive_gaussian_2d (reference src/igs/gs2d.py:24-44):
 *   q = A dx^2 + 2 B dx dy + D dy^2, w = alpha exp(-q/2), out_c = sum w c / (sum w + eps).
 * Backward is the derivative of that expression by the quotient rule, accumulated pair by
 * pair (no factoring shared with the Python oracle's vectorised form):
 *   d out_c / d w_n = (c_nc - out_c) / (den + eps).
 *
 * Build: gcc -O2 -shared -fPIC -o oracle/libgs2d_bruteforce.so oracle/gs2d_bruteforce.c -lm
 */
#include <math.h>
#include <stddef.h>

/* x,y: [B,H,W]; pos: [B,N,2]; A,Bc,D,alpha: [B,N]; col: [B,N,C]; out: [B,C,H,W]; den: [B,H,W] */
void gs2d_bf_forward(const double *x, const double *y, const double *pos, const double *A,
                     const double *Bc, const double *D, const double *alpha, const double *col,
                     int B, int N, int H, int W, int C, double eps, double *out, double *den)
{
    for (int b = 0; b < B; ++b)
        for (int p = 0; p < H * W; ++p) {
            double xv = x[(size_t)b * H * W + p], yv = y[(size_t)b * H * W + p];
            double s = 0.0;
            for (int c = 0; c < C; ++c) out[((size_t)b * C + c) * H * W + p] = 0.0;
            for (int n = 0; n < N; ++n) {
                size_t bn = (size_t)b * N + n;
                double dx = xv - pos[2 * bn], dy = yv - pos[2 * bn + 1];
                double q = A[bn] * dx * dx + 2.0 * Bc[bn] * dx * dy + D[bn] * dy * dy;
                double w = alpha[bn] * exp(-0.5 * q);
                s += w;
                for (int c = 0; c < C; ++c) out[((size_t)b * C + c) * H * W + p] += w * col[bn * C + c];
            }
            den[(size_t)b * H * W + p] = s;
            for (int c = 0; c < C; ++c) out[((size_t)b * C + c) * H * W + p] /= (s + eps);
        }
}

/* gout: [B,C,H,W]; out/den from the forward.  All gradient arrays must be zeroed by the
 * caller.  gx, gy may be NULL. */
void gs2d_bf_backward(const double *x, const double *y, const double *pos, const double *A,
                      const double *Bc, const double *D, const double *alpha, const double *col,
                      const double *out, const double *den, const double *gout,
                      int B, int N, int H, int W, int C, double eps,
                      double *gpos, double *gA, double *gB, double *gD, double *galpha,
                      double *gcol, double *gx, double *gy)
{
    for (int b = 0; b < B; ++b)
        for (int p = 0; p < H * W; ++p) {
            size_t bp = (size_t)b * H * W + p;
            double xv = x[bp], yv = y[bp], S = den[bp] + eps;
            for (int n = 0; n < N; ++n) {
                size_t bn = (size_t)b * N + n;
                double dx = xv - pos[2 * bn], dy = yv - pos[2 * bn + 1];
                double q = A[bn] * dx * dx + 2.0 * Bc[bn] * dx * dy + D[bn] * dy * dy;
                double e = exp(-0.5 * q), w = alpha[bn] * e;
                double dLdw = 0.0; /* sum_c gout_c * d out_c / d w_n */
                for (int c = 0; c < C; ++c) {
                    double g = gout[((size_t)b * C + c) * H * W + p];
                    double o = out[((size_t)b * C + c) * H * W + p];
                    dLdw += g * (col[bn * C + c] - o) / S;
                    gcol[bn * C + c] += g * w / S;
                }
                galpha[bn] += dLdw * e;
                double dLdq = dLdw * w * (-0.5);
                gA[bn] += dLdq * dx * dx;
                gB[bn] += dLdq * 2.0 * dx * dy;
                gD[bn] += dLdq * dy * dy;
                double dqdx = 2.0 * A[bn] * dx + 2.0 * Bc[bn] * dy;
                double dqdy = 2.0 * Bc[bn] * dx + 2.0 * D[bn] * dy;
                gpos[2 * bn] -= dLdq * dqdx;
                gpos[2 * bn + 1] -= dLdq * dqdy;
                if (gx) gx[bp] += dLdq * dqdx;
                if (gy) gy[bp] += dLdq * dqdy;
            }
        }
}
