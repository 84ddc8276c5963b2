// Projections with FEW rows (the pooled features of a batch: one row per crystal).  The library GEMM
// the framework calls runs such a product on one or two workgroups (20 us for 256 x 128 x 128); here a
// wavefront owns a 32x32 block of the result, so even 256 rows give dozens of wavefronts, and bias,
// rectifier and the layout of the weight (O, I) as torch.nn.Linear stores it are handled in place.
//   forward   y (M,N) = x (M,K) W^T + b, W (N,K)           (reference: torch.nn.functional.linear)
//   backward  dx (M,K) = dy (M,N) W
#pragma once
#include "device_common.hpp"

namespace cfh {

typedef float v4f_g __attribute__((ext_vector_type(4)));

// lane (kk, col) of a wavefront: A operand A[m = col][k = kk], B operand B[k = kk][n = col]; a 16-wide step
// of the reduction index is four MFMA 16x16x4 with k = 4 kk + j, j = 0..3, so that a lane reads 4
// consecutive floats of its row.
// grid: (ceil(M/64), ceil(N/64)), block 256 = 4 wavefronts, wavefront w: rows 32 (w/2), columns 32 (w%2).
// K % 16 == 0, rows 16-byte aligned.
__global__ __launch_bounds__(256) void small_linear_fwd_kernel(const float* __restrict__ x, const float* __restrict__ w,
                                                               const float* __restrict__ b, float* __restrict__ y,
                                                               int M, int N, int K, int relu) {
    const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
    const int col = lane & 15, kk = lane >> 4;
    const int m0 = blockIdx.x * 64 + 32 * (wv >> 1), n0 = blockIdx.y * 64 + 32 * (wv & 1);
    if (m0 >= M || n0 >= N) return;
    const int ra = min(m0 + col, M - 1), rb = min(m0 + 16 + col, M - 1);
    const int ca = min(n0 + col, N - 1), cb = min(n0 + 16 + col, N - 1);
    const float4* xa = reinterpret_cast<const float4*>(x + (size_t)ra * K) + kk;
    const float4* xb = reinterpret_cast<const float4*>(x + (size_t)rb * K) + kk;
    const float4* wa = reinterpret_cast<const float4*>(w + (size_t)ca * K) + kk;
    const float4* wb = reinterpret_cast<const float4*>(w + (size_t)cb * K) + kk;
    v4f_g acc00 = {0.f, 0.f, 0.f, 0.f}, acc01 = acc00, acc10 = acc00, acc11 = acc00;
    const int chunks = K / 16;
    auto products = [&](const float4& a0, const float4& a1, const float4& b0, const float4& b1) {
        const float A0[4] = {a0.x, a0.y, a0.z, a0.w}, A1[4] = {a1.x, a1.y, a1.z, a1.w};
        const float B0[4] = {b0.x, b0.y, b0.z, b0.w}, B1[4] = {b1.x, b1.y, b1.z, b1.w};
#pragma unroll
        for (int j = 0; j < 4; j++) {
            acc00 = __builtin_amdgcn_mfma_f32_16x16x4f32(A0[j], B0[j], acc00, 0, 0, 0);
            acc01 = __builtin_amdgcn_mfma_f32_16x16x4f32(A0[j], B1[j], acc01, 0, 0, 0);
            acc10 = __builtin_amdgcn_mfma_f32_16x16x4f32(A1[j], B0[j], acc10, 0, 0, 0);
            acc11 = __builtin_amdgcn_mfma_f32_16x16x4f32(A1[j], B1[j], acc11, 0, 0, 0);
        }
    };
    // four chunks at a time, their sixteen loads asked for before the first product (left to itself the compiler puts
    // every load next to its product: a chain of trips to the L2, and the kernel is nothing but that chain)
    int c = 0;
    for (; c + 4 <= chunks; c += 4) {
        float4 a0[4], a1[4], b0[4], b1[4];
#pragma unroll
        for (int u = 0; u < 4; u++) { a0[u] = xa[4 * (c + u)]; a1[u] = xb[4 * (c + u)]; b0[u] = wa[4 * (c + u)]; b1[u] = wb[4 * (c + u)]; }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int u = 0; u < 4; u++) products(a0[u], a1[u], b0[u], b1[u]);
    }
    for (; c < chunks; c++) products(xa[4 * c], xb[4 * c], wa[4 * c], wb[4 * c]);
    // accumulator component c of lane (kk, col): row 4 kk + c of the 16x16 block, column col
    const float ba = b ? b[ca] : 0.f, bb = b ? b[cb] : 0.f;
    auto put = [&](int r, int n, float v) {
        if (r < M && n < N) y[(size_t)r * N + n] = relu ? fmaxf(v, 0.f) : v;
    };
#pragma unroll
    for (int c = 0; c < 4; c++) {
        const int r0 = m0 + 4 * kk + c;
        put(r0, n0 + col, acc00[c] + ba);
        put(r0, n0 + 16 + col, acc01[c] + bb);
        put(r0 + 16, n0 + col, acc10[c] + ba);
        put(r0 + 16, n0 + 16 + col, acc11[c] + bb);
    }
}

// dx (M,K) = dy (M,N) W, W (N,K).  grid: (ceil(M/64), ceil(K/64)); N % 16 == 0, rows of dy 16-byte aligned.
__global__ __launch_bounds__(256) void small_linear_dx_kernel(const float* __restrict__ dy, const float* __restrict__ w,
                                                              float* __restrict__ dx, int M, int N, int K) {
    const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
    const int col = lane & 15, kk = lane >> 4;
    const int m0 = blockIdx.x * 64 + 32 * (wv >> 1), k0 = blockIdx.y * 64 + 32 * (wv & 1);
    if (m0 >= M || k0 >= K) return;
    const int ra = min(m0 + col, M - 1), rb = min(m0 + 16 + col, M - 1);
    const int ca = min(k0 + col, K - 1), cb = min(k0 + 16 + col, K - 1);
    const float4* ya = reinterpret_cast<const float4*>(dy + (size_t)ra * N) + kk;
    const float4* yb = reinterpret_cast<const float4*>(dy + (size_t)rb * N) + kk;
    v4f_g acc00 = {0.f, 0.f, 0.f, 0.f}, acc01 = acc00, acc10 = acc00, acc11 = acc00;
    const int chunks = N / 16;
    // two chunks at a time, all their loads asked for before the first product (see small_linear_fwd_kernel)
    auto step = [&](int c, int nch) {
        float4 a0[2], a1[2];
        float b0[2][4], b1[2][4];
#pragma unroll
        for (int u = 0; u < 2; u++) {
            const int cu = u < nch ? c + u : c;
            a0[u] = ya[4 * cu]; a1[u] = yb[4 * cu];
#pragma unroll
            for (int j = 0; j < 4; j++) {
                const float* wr = w + (size_t)(16 * cu + 4 * kk + j) * K;      // row n = 16 c + 4 kk + j of W
                b0[u][j] = wr[ca]; b1[u][j] = wr[cb];
            }
        }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int u = 0; u < 2; u++) {
            if (u >= nch) continue;
            const float A0[4] = {a0[u].x, a0[u].y, a0[u].z, a0[u].w}, A1[4] = {a1[u].x, a1[u].y, a1[u].z, a1[u].w};
#pragma unroll
            for (int j = 0; j < 4; j++) {
                acc00 = __builtin_amdgcn_mfma_f32_16x16x4f32(A0[j], b0[u][j], acc00, 0, 0, 0);
                acc01 = __builtin_amdgcn_mfma_f32_16x16x4f32(A0[j], b1[u][j], acc01, 0, 0, 0);
                acc10 = __builtin_amdgcn_mfma_f32_16x16x4f32(A1[j], b0[u][j], acc10, 0, 0, 0);
                acc11 = __builtin_amdgcn_mfma_f32_16x16x4f32(A1[j], b1[u][j], acc11, 0, 0, 0);
            }
        }
    };
    int c = 0;
    for (; c + 2 <= chunks; c += 2) step(c, 2);
    if (c < chunks) step(c, 1);
    auto put = [&](int r, int n, float v) {
        if (r < M && n < K) dx[(size_t)r * K + n] = v;
    };
#pragma unroll
    for (int c = 0; c < 4; c++) {
        const int r0 = m0 + 4 * kk + c;
        put(r0, k0 + col, acc00[c]);
        put(r0, k0 + 16 + col, acc01[c]);
        put(r0 + 16, k0 + col, acc10[c]);
        put(r0 + 16, k0 + 16 + col, acc11[c]);
    }
}

// The same for a few output features (N not a multiple of 16, e.g. the single regression target): one thread per
// element of dx, the N terms in a loop.  grid: ceil(M K / 256) blocks of 256 threads.
__global__ __launch_bounds__(256) void small_linear_dx_narrow_kernel(const float* __restrict__ dy, const float* __restrict__ w,
                                                                     float* __restrict__ dx, int M, int N, int K) {
    const long idx = (long)blockIdx.x * 256 + threadIdx.x;
    if (idx >= (long)M * K) return;
    const int m = (int)(idx / K), k = (int)(idx - (long)m * K);
    float acc = 0.0f;
    for (int n = 0; n < N; n++) acc = fmaf(dy[(size_t)m * N + n], w[(size_t)n * K + k], acc);
    dx[idx] = acc;
}

}  // namespace cfh
