// What sits between the stacked q/k/v projection of a layer and its lattice-sum / attention kernels,
// in one launch each way: split of the projection output into query, key and value, the query
// scaled by 1/sqrt(Dh), and the Gaussian coefficient of every (atom, head)
//     alpha = q_h . w_h,  alpha' = (alpha + shift) scale,  a = ((1 - lb) elu(c1 alpha') + 1) c2
// (reference: models/indexed_lattice_multi_head_attention_cuda.py:896-940 and the query scaling of
// :144-185, there a dozen elementwise launches of the framework per direction).
// Lane layout: thread = (atom, channel c = h Dh + d) with Dh = 16, so the 16 lanes of a DPP row are
// the channels of one head and the dot product is a row reduction.
#pragma once
#include "device_common.hpp"

namespace cfh {

struct AttnInArgs {
    const float* qkv;          // (N, 3 HD): query, key, value blocks of a row
    const float* w;            // (HD) lattice_pos_weights
    const float* gauss;        // device {scale, shift} or null
    const float* gqs;          // backward inputs, (N, HD) each, (N, H) for ga; any may be null (= zero)
    const float* gk;
    const float* gv;
    const float* ga;
    float* qs;                 // forward outputs
    float* k;
    float* v;
    float* a;
    float* gqkv;               // backward outputs: (N, 3 HD) and (HD)
    float* gw;
    float* partial;            // backward scratch: (blocks, HD) per-block sums of the weight gradient
    int N, HD, rows_per_block;
    float c1, lb, c2, q_scale;
};

__device__ __forceinline__ float gauss_alpha(const AttnInArgs& P, float q, float wc, float& slope) {
    float alpha = row_sum(q * wc);
    float scale = 1.0f;
    if (P.gauss) {
        scale = P.gauss[0];
        alpha = (alpha + P.gauss[1]) * scale;
    }
    const float u = alpha * P.c1;
    const float e = u > 0.0f ? u : expm1f(u);
    slope = (u > 0.0f ? 1.0f : e + 1.0f) * P.c1 * scale * (1.0f - P.lb) * P.c2;      // da / d(q.w)
    return ((1.0f - P.lb) * e + 1.0f) * P.c2;
}

// grid: ceil(N HD / 256) blocks of 256 threads
__global__ __launch_bounds__(256) void attention_inputs_fwd_kernel(AttnInArgs P) {
    const long idx = (long)blockIdx.x * 256 + threadIdx.x;
    const int n = (int)(idx / P.HD), c = (int)(idx - (long)n * P.HD);
    const bool live = n < P.N;
    const float* row = P.qkv + (size_t)(live ? n : 0) * 3 * P.HD;
    const float q = live ? row[c] : 0.0f;
    float slope;
    const float a = gauss_alpha(P, q, P.w[c], slope);
    if (!live) return;
    const size_t o = (size_t)n * P.HD + c;
    P.qs[o] = q * P.q_scale;
    P.k[o] = row[P.HD + c];
    P.v[o] = row[2 * P.HD + c];
    if ((c & 15) == 0) P.a[(size_t)n * (P.HD >> 4) + (c >> 4)] = a;
}

// grid: ceil(N / rows_per_block) blocks of 256 threads; 256 % HD == 0.  Thread = (row offset, channel),
// walks rows_per_block rows in steps of 256 / HD; the block's sum of the weight gradient goes to
// partial[block][HD] (no atomics: a second small launch adds the blocks up).
__global__ __launch_bounds__(256) void attention_inputs_bwd_kernel(AttnInArgs P) {
    const int c = threadIdx.x % P.HD, r = threadIdx.x / P.HD, step = 256 / P.HD;
    const int n0 = blockIdx.x * P.rows_per_block;
    const int n1 = min(P.N, n0 + P.rows_per_block);
    const float wc = P.w[c];
    const int H = P.HD >> 4;
    float gw = 0.0f;
#pragma unroll 4
    for (int nb = n0; nb < n0 + P.rows_per_block; nb += step) {   // uniform trip count: row_sum needs every lane
        const int n = nb + r;
        const bool live = n < n1;
        const size_t row = (size_t)(live ? n : n0) * 3 * P.HD;
        const size_t o = (size_t)(live ? n : n0) * P.HD + c;
        const float q = P.qkv[row + c];
        const float ga = P.ga ? P.ga[(size_t)(live ? n : n0) * H + (c >> 4)] : 0.0f;
        const float gqs = P.gqs ? P.gqs[o] : 0.0f;
        const float gk = P.gk ? P.gk[o] : 0.0f;
        const float gv = P.gv ? P.gv[o] : 0.0f;
        float slope;
        gauss_alpha(P, q, wc, slope);
        const float galpha = ga * slope;
        if (live) {
            gw += galpha * q;
            P.gqkv[row + c] = galpha * wc + gqs * P.q_scale;
            P.gqkv[row + P.HD + c] = gk;
            P.gqkv[row + 2 * P.HD + c] = gv;
        }
    }
    __shared__ float part[256];
    part[threadIdx.x] = gw;
    __syncthreads();
    if (threadIdx.x < P.HD) {
        float sum = 0.0f;
        for (int g = 0; g < step; g++) sum += part[threadIdx.x + g * P.HD];
        P.partial[(size_t)blockIdx.x * P.HD + threadIdx.x] = sum;
    }
}

// gw[c] = sum over blocks of partial[block][c].  grid: ceil(HD / 32) blocks of 1024 threads = 32 groups x 32 channels
__global__ __launch_bounds__(1024) void attention_inputs_gw_kernel(const float* __restrict__ partial, int nblocks, int HD,
                                                                   float* __restrict__ gw) {
    const int c = blockIdx.x * 32 + (threadIdx.x & 31), g = threadIdx.x >> 5;
    float sum = 0.0f;
    if (c < HD)
        for (int b = g; b < nblocks; b += 32) sum += partial[(size_t)b * HD + c];
    __shared__ float part[1024];
    part[threadIdx.x] = sum;
    __syncthreads();
    if (g == 0 && c < HD) {
        float total = 0.0f;
        for (int k = 0; k < 32; k++) total += part[(threadIdx.x & 31) + 32 * k];
        gw[c] = total;
    }
}

}  // namespace cfh
