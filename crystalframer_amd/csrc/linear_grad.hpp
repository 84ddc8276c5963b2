// Weight and bias gradients of y = x W^T + b for the projections around the attention
// (N rows = atoms, a few hundred columns):  dW (O,I) = dY^T X,  db (O) = sum over rows of dY.
// The library GEMM the framework would call picks a 32x32 tile without splitting the long
// dimension for these shapes (16 workgroups for a 128x128 output, 19 us) and the bias gradient is
// a second launch; here the N rows are split over gridDim.z slices so that a launch fills the chip,
// each wavefront owns a 32x32 block of dW as four v_mfma_f32_16x16x4 accumulators, and the slices
// are combined with float atomics into the zeroed outputs (so the sum order, and the last bits,
// can differ from run to run).
#pragma once
#include "device_common.hpp"

namespace cfh {

typedef float v4f_l __attribute__((ext_vector_type(4)));

// One workgroup's share: 256 threads = 4 wavefronts, wavefront w owns the 32x32 block
// (64 ty + 32 (w/2), 64 tx + 32 (w%2)) of dW and the rows [slice rows_per_slice, ...) of x and dy
// (row strides ldx, ldy: dy may be a column slice of a wider matrix).  dW == nullptr: only db is
// computed (x is not read; I = 1).
__device__ __forceinline__ void wgrad_block(const float* __restrict__ x, const float* __restrict__ dy, int N, int I,
                                            int O, int ldx, int ldy, int rows_per_slice, int tx, int ty, int slice,
                                            float* dW, float* db) {
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
    const int o0 = ty * 64 + 32 * (w >> 1);
    const int i0 = tx * 64 + 32 * (w & 1);
    if (o0 >= O || i0 >= I) return;
    const int r0 = slice * rows_per_slice;
    const int r1 = min(N, r0 + rows_per_slice);
    const int col = lane & 15, kk = lane >> 4;
    const int oa = o0 + col, ob = o0 + 16 + col;          // columns of dY this lane feeds (A operand)
    const int ia = i0 + col, ib = i0 + 16 + col;          // columns of X this lane feeds (B operand)
    const bool has_w = dW != nullptr;                     // no dW: the column sums of dY alone
    const bool voa = oa < O, vob = ob < O, via = has_w && ia < I, vib = has_w && ib < I;
    v4f_l acc00 = {0.f, 0.f, 0.f, 0.f}, acc01 = acc00, acc10 = acc00, acc11 = acc00;
    float bsum_a = 0.f, bsum_b = 0.f;
#pragma unroll 4
    for (int r = r0 + kk; r < r1 + kk; r += 4) {          // every lane group takes the same number of steps
        const bool vr = r < r1;
        const float ya = (vr && voa) ? dy[(size_t)r * ldy + oa] : 0.f;
        const float yb = (vr && vob) ? dy[(size_t)r * ldy + ob] : 0.f;
        const float xa = (vr && via) ? x[(size_t)r * ldx + ia] : 0.f;
        const float xb = (vr && vib) ? x[(size_t)r * ldx + ib] : 0.f;
        acc00 = __builtin_amdgcn_mfma_f32_16x16x4f32(ya, xa, acc00, 0, 0, 0);
        acc01 = __builtin_amdgcn_mfma_f32_16x16x4f32(ya, xb, acc01, 0, 0, 0);
        acc10 = __builtin_amdgcn_mfma_f32_16x16x4f32(yb, xa, acc10, 0, 0, 0);
        acc11 = __builtin_amdgcn_mfma_f32_16x16x4f32(yb, xb, acc11, 0, 0, 0);
        bsum_a += ya; bsum_b += yb;
    }
    // accumulator component c of lane (kk, col): row 4 kk + c of the 16x16 block, column col
#pragma unroll
    for (int c = 0; c < 4; c++) {
        const int oo = 4 * kk + c;
        if (o0 + oo < O) {
            if (via) atomicAdd(dW + (size_t)(o0 + oo) * I + ia, acc00[c]);
            if (vib) atomicAdd(dW + (size_t)(o0 + oo) * I + ib, acc01[c]);
        }
        if (o0 + 16 + oo < O) {
            if (via) atomicAdd(dW + (size_t)(o0 + 16 + oo) * I + ia, acc10[c]);
            if (vib) atomicAdd(dW + (size_t)(o0 + 16 + oo) * I + ib, acc11[c]);
        }
    }
    if (db && tx == 0 && (w & 1) == 0) {                  // one column of blocks sums dY over its rows
        bsum_a = rows_sum(bsum_a);
        bsum_b = rows_sum(bsum_b);
        if (kk == 0) {
            if (voa) atomicAdd(db + oa, bsum_a);
            if (vob) atomicAdd(db + ob, bsum_b);
        }
    }
}

// grid: (ceil(I/64), ceil(O/64), slices), block: 256 threads
__global__ __launch_bounds__(256) void linear_wgrad_kernel(const float* __restrict__ x, const float* __restrict__ dy,
                                                           int N, int I, int O, int rows_per_slice,
                                                           float* dW, float* db) {
    wgrad_block(x, dy, N, I, O, I, O, rows_per_slice, blockIdx.x, blockIdx.y, blockIdx.z, dW, db);
}

// Several layers' gradients in one launch: the jobs travel in the kernel arguments, workgroup b
// belongs to the job with block0 <= b < block0 + bx by slices.
constexpr int WGRAD_MAX_JOBS = 32;
struct WgradJob {
    const float* x; const float* dy; float* dW; float* db;
    int N, I, O, ldx, ldy;
    int block0, bx, by, rows_per_slice;
};
struct WgradJobs { WgradJob job[WGRAD_MAX_JOBS]; int njobs; };

__global__ __launch_bounds__(256) void linear_wgrad_batch_kernel(const WgradJobs T) {
    int j = 0;
    for (int t = 1; t < T.njobs; t++)
        if ((int)blockIdx.x >= T.job[t].block0) j = t;
    const WgradJob& J = T.job[j];
    const int b = (int)blockIdx.x - J.block0;
    const int tiles = J.bx * J.by;
    const int slice = b / tiles, tile = b - slice * tiles;
    wgrad_block(J.x, J.dy, J.N, J.I, J.O, J.ldx, J.ldy, J.rows_per_slice, tile % J.bx, tile / J.bx, slice, J.dW, J.db);
}

__global__ __launch_bounds__(256) void zero2_kernel(float* a, int na, float* b, int nb) {
    const int idx = blockIdx.x * blockDim.x + threadIdx.x;
    if (idx < na) a[idx] = 0.0f;
    if (b && idx < nb) b[idx] = 0.0f;
}

}  // namespace cfh
