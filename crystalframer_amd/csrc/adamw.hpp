// AdamW update of many parameter tensors in one launch (decoupled weight decay, bias correction; the update rule of
// torch.optim.AdamW without amsgrad / maximize).  The job table travels in the kernel arguments; a block of 256
// threads takes 1024 consecutive elements of one tensor.  The number of steps taken so far lives in device memory
// (so that a captured launch advances from replay to replay) and is advanced by a second, one-thread launch.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace cfh {

constexpr int ADAMW_MAX_JOBS = 80;
constexpr int ADAMW_BLOCK_ELEMS = 1024;

struct AdamWJob {
    float* p;
    const float* g;
    float* m;
    float* v;
    int n;
    int block0;       // first block of this tensor
};
struct AdamWJobs {
    AdamWJob job[ADAMW_MAX_JOBS];
    int njobs;
    float lr, beta1, beta2, eps, wd;
    const unsigned long long* step;      // steps taken before this one
};

__device__ __forceinline__ void adamw_element(float& p, float g, float& m, float& v, float decay, float b1, float b2,
                                              float step_size, float inv_sqrt_bc2, float eps) {
    p *= decay;
    m = fmaf(b1, m, (1.0f - b1) * g);
    v = fmaf(b2, v, (1.0f - b2) * g * g);
    const float denom = fmaf(sqrtf(v), inv_sqrt_bc2, eps);
    p -= step_size * (m / denom);
}

__global__ __launch_bounds__(256) void adamw_batch_kernel(const AdamWJobs T) {
    const int b = (int)blockIdx.x;
    int lo = 0, hi = T.njobs;            // job[lo].block0 <= b < job[hi].block0
    while (hi - lo > 1) {
        const int mid = (lo + hi) >> 1;
        if (T.job[mid].block0 <= b) lo = mid; else hi = mid;
    }
    const AdamWJob J = T.job[lo];
    const float t = (float)(*T.step + 1ULL);
    // 1 - beta^t in double: for beta close to 1 and the first steps the float form cancels (1 - 0.999 has three digits)
    const float bc1 = (float)(-expm1((double)t * log((double)T.beta1)));
    const float bc2 = (float)(-expm1((double)t * log((double)T.beta2)));
    const float step_size = T.lr / bc1;
    const float inv_sqrt_bc2 = rsqrtf(bc2);
    const float decay = 1.0f - T.lr * T.wd;
    const int base = (b - J.block0) * ADAMW_BLOCK_ELEMS + (int)threadIdx.x * 4;
    if (base >= J.n) return;
    const bool vec = base + 4 <= J.n &&
                     ((((uintptr_t)J.p) | ((uintptr_t)J.g) | ((uintptr_t)J.m) | ((uintptr_t)J.v)) & 15) == 0;
    if (vec) {
        float4 p = *reinterpret_cast<const float4*>(J.p + base);
        const float4 g = *reinterpret_cast<const float4*>(J.g + base);
        float4 m = *reinterpret_cast<const float4*>(J.m + base);
        float4 v = *reinterpret_cast<const float4*>(J.v + base);
        adamw_element(p.x, g.x, m.x, v.x, decay, T.beta1, T.beta2, step_size, inv_sqrt_bc2, T.eps);
        adamw_element(p.y, g.y, m.y, v.y, decay, T.beta1, T.beta2, step_size, inv_sqrt_bc2, T.eps);
        adamw_element(p.z, g.z, m.z, v.z, decay, T.beta1, T.beta2, step_size, inv_sqrt_bc2, T.eps);
        adamw_element(p.w, g.w, m.w, v.w, decay, T.beta1, T.beta2, step_size, inv_sqrt_bc2, T.eps);
        *reinterpret_cast<float4*>(J.p + base) = p;
        *reinterpret_cast<float4*>(J.m + base) = m;
        *reinterpret_cast<float4*>(J.v + base) = v;
    } else {
        for (int u = base; u < min(base + 4, J.n); u++) {
            float p = J.p[u], m = J.m[u], v = J.v[u];
            adamw_element(p, J.g[u], m, v, decay, T.beta1, T.beta2, step_size, inv_sqrt_bc2, T.eps);
            J.p[u] = p; J.m[u] = m; J.v[u] = v;
        }
    }
}

__global__ void adamw_advance_kernel(unsigned long long* step) { *step += 1ULL; }

}  // namespace cfh
