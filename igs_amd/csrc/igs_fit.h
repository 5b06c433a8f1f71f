// igs_fit.h -- AdamW step of the fused fit iteration.
// Included by igs_gs2d.hip inside its anonymous namespace (one translation unit).
#pragma once

// ----------------------------------------------------------------------------- AdamW
// Decoupled-weight-decay Adam over one flat parameter block, the update of torch.optim.AdamW
// (amsgrad off) as the fit script configures it (scripts/2dgs_img_comp.py:186-193).  The
// step counter and learning rate live in device memory so that a captured graph advances:
//   state = {lr, t, 1 - beta1^t, sqrt(1 - beta2^t), ticket, -, -, -}; lr is written by the host.
// Every workgroup reads t, forms the bias corrections of step t + 1 (one thread, powers in double)
// and updates its elements; the workgroup that finishes last (integer ticket, zero before and after
// the launch) writes t + 1 and the corrections back, when no workgroup needs the old t any more.
constexpr int kAdamStateFloats = 8;
__global__ __launch_bounds__(kThreads) void k_adamw(float* __restrict__ param,
                                                    const float* __restrict__ grad,
                                                    float* __restrict__ exp_avg,
                                                    float* __restrict__ exp_avg_sq, long n,
                                                    float* __restrict__ state, float beta1,
                                                    float beta2, float eps, float weight_decay) {
    __shared__ float corr[3];  // t + 1, 1 - beta1^(t+1), sqrt(1 - beta2^(t+1))
    if (threadIdx.x == 0) {
        const float t = state[1] + 1.0f;
        corr[0] = t;
        corr[1] = (float)(1.0 - pow((double)beta1, (double)t));
        corr[2] = (float)sqrt(1.0 - pow((double)beta2, (double)t));
    }
    __syncthreads();
    const long i = (long)blockIdx.x * kThreads + threadIdx.x;
    if (i < n) {
        const float lr = state[0], bc1 = corr[1], bc2_sqrt = corr[2];
        const float g = grad[i];
        float p = param[i] * (1.0f - lr * weight_decay);
        float m = exp_avg[i];
        m = fmaf(g - m, 1.0f - beta1, m);
        const float v = fmaf(g * g, 1.0f - beta2, exp_avg_sq[i] * beta2);
        const float denom = sqrtf(v) / bc2_sqrt + eps;
        p -= (lr / bc1) * (m / denom);
        param[i] = p;
        exp_avg[i] = m;
        exp_avg_sq[i] = v;
    }
    __syncthreads();  // every thread of the workgroup has read what it needs of `state`
    if (threadIdx.x == 0) {
        unsigned int* ticket = reinterpret_cast<unsigned int*>(state + 4);
        if (atomicAdd(ticket, 1u) == gridDim.x - 1u) {  // every workgroup has read t
            state[1] = corr[0];
            state[2] = corr[1];
            state[3] = corr[2];
            *ticket = 0u;
        }
    }
}

// ----------------------------------------------------------------------------- position penalty
// Regulariser of the fit loop (scripts/2dgs_img_comp.py:224-228): weight * mean(relu(|p| - 1)) over
// the position columns (the first two floats of every row of `rows` x `stride` floats).  Every
// thread adds the gradient weight * sign(p) [|p| > 1] / count of its row to g_feature; workgroup 0
// also sums the penalty over all rows in a fixed order and adds it to loss[0].
__global__ __launch_bounds__(kThreads) void k_position_penalty(const float* __restrict__ feature, long rows,
                                                               int stride, float weight, float inv_count,
                                                               float* __restrict__ g_feature,
                                                               float* __restrict__ loss) {
    const long r = (long)blockIdx.x * kThreads + threadIdx.x;
    if (r < rows) {
#pragma unroll
        for (int k = 0; k < 2; ++k) {
            const float p = feature[r * stride + k];
            if (fabsf(p) > 1.0f) g_feature[r * stride + k] += copysignf(weight * inv_count, p);
        }
    }
    if (blockIdx.x != 0 || loss == nullptr) return;  // workgroup-uniform
    __shared__ float red[kThreads];
    float s = 0.0f;
    for (long i = threadIdx.x; i < rows; i += kThreads) {
        s += fmaxf(fabsf(feature[i * stride]) - 1.0f, 0.0f);
        s += fmaxf(fabsf(feature[i * stride + 1]) - 1.0f, 0.0f);
    }
    red[threadIdx.x] = s;
    __syncthreads();
    for (int k = kThreads / 2; k > 0; k >>= 1) {
        if ((int)threadIdx.x < k) red[threadIdx.x] += red[threadIdx.x + k];
        __syncthreads();
    }
    if (threadIdx.x == 0) loss[0] += weight * inv_count * red[0];
}
