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
    if (r1 <= r0) return;
    const int col = lane & 15, kk = lane >> 4;
    const int oa = o0 + col, ob = o0 + 16 + col;          // columns of dY this lane feeds (A operand)
    const int ia = i0 + col, ib = i0 + 16 + col;          // columns of X this lane feeds (B operand)
    const bool has_w = dW != nullptr;                     // no dW: the column sums of dY alone
    const bool voa = oa < O, vob = ob < O, via = has_w && ia < I, vib = has_w && ib < I;
    // Every load is unconditional: a column past the edge reads the first column of the block instead (its products
    // land in accumulator rows / columns that are not written), a row past the end of the slice reads the first row of
    // its chunk and its dY is set to zero.  Without dW the B operand mirrors dY (the products are not used).
    const float* const xs = has_w ? x : dy;
    const int lx = has_w ? ldx : ldy;
    const uint32_t cya = 4u * (uint32_t)(voa ? oa : o0), cyb = 4u * (uint32_t)(vob ? ob : o0);
    const uint32_t cxa = 4u * (uint32_t)(via ? ia : (has_w ? i0 : 0)), cxb = 4u * (uint32_t)(vib ? ib : (has_w ? i0 : 0));
    constexpr int UN = 4;                                 // steps of four rows per chunk
    uint32_t oy[UN], ox[UN];                              // byte offsets of the lane's rows within a chunk
#pragma unroll
    for (int u = 0; u < UN; u++) {
        oy[u] = 4u * (uint32_t)(kk + 4 * u) * (uint32_t)ldy;
        ox[u] = 4u * (uint32_t)(kk + 4 * u) * (uint32_t)lx;
    }
    const char* by = reinterpret_cast<const char*>(dy + (size_t)r0 * ldy);      // the chunk's first row (uniform)
    const char* bx = reinterpret_cast<const char*>(xs + (size_t)r0 * lx);
    const size_t sy = (size_t)4 * UN * 4 * ldy, sx = (size_t)4 * UN * 4 * lx;   // bytes per chunk
    v4f_l acc00 = {0.f, 0.f, 0.f, 0.f}, acc01 = acc00, acc10 = acc00, acc11 = acc00;
    float bsum_a = 0.f, bsum_b = 0.f;
    auto ld = [](const char* base, uint32_t off) { return *reinterpret_cast<const float*>(base + off); };
    auto products = [&](const float (&ya)[UN], const float (&yb)[UN], const float (&xa)[UN], const float (&xb)[UN]) {
#pragma unroll
        for (int u = 0; u < UN; u++) {
            acc00 = __builtin_amdgcn_mfma_f32_16x16x4f32(ya[u], xa[u], acc00, 0, 0, 0);
            acc01 = __builtin_amdgcn_mfma_f32_16x16x4f32(ya[u], xb[u], acc01, 0, 0, 0);
            acc10 = __builtin_amdgcn_mfma_f32_16x16x4f32(yb[u], xa[u], acc10, 0, 0, 0);
            acc11 = __builtin_amdgcn_mfma_f32_16x16x4f32(yb[u], xb[u], acc11, 0, 0, 0);
            bsum_a += ya[u]; bsum_b += yb[u];
        }
    };
    // whole chunks of 16 rows; the loads of the next chunk are asked for before the products of this one (the rows
    // come from beyond the L2 more often than not, and seven wavefronts a SIMD with sixteen loads each in flight did
    // not cover that)
    const int nfull = (r1 - r0) / (4 * UN);
    if (nfull > 0) {
        float ya[UN], yb[UN], xa[UN], xb[UN];
#pragma unroll
        for (int u = 0; u < UN; u++) {
            ya[u] = ld(by, oy[u] + cya); yb[u] = ld(by, oy[u] + cyb);
            xa[u] = ld(bx, ox[u] + cxa); xb[u] = ld(bx, ox[u] + cxb);
        }
        for (int c = 1; c < nfull; c++) {
            by += sy; bx += sx;
            float na[UN], nb[UN], ma[UN], mb[UN];
#pragma unroll
            for (int u = 0; u < UN; u++) {
                na[u] = ld(by, oy[u] + cya); nb[u] = ld(by, oy[u] + cyb);
                ma[u] = ld(bx, ox[u] + cxa); mb[u] = ld(bx, ox[u] + cxb);
            }
            products(ya, yb, xa, xb);
#pragma unroll
            for (int u = 0; u < UN; u++) { ya[u] = na[u]; yb[u] = nb[u]; xa[u] = ma[u]; xb[u] = mb[u]; }
        }
        products(ya, yb, xa, xb);
        by += sy; bx += sx;
    }
    const int rt = r0 + 4 * UN * nfull;                   // the rows left: fewer than a chunk
    if (rt < r1) {
        float ya[UN], yb[UN], xa[UN], xb[UN];
#pragma unroll
        for (int u = 0; u < UN; u++) {
            const bool vr = rt + kk + 4 * u < r1;
            const uint32_t qy = vr ? oy[u] : 0u, qx = vr ? ox[u] : 0u;
            ya[u] = ld(by, qy + cya); yb[u] = ld(by, qy + cyb);
            xa[u] = ld(bx, qx + cxa); xb[u] = ld(bx, qx + cxb);
            ya[u] = vr ? ya[u] : 0.f; yb[u] = vr ? yb[u] : 0.f;
        }
        products(ya, yb, xa, xb);
    }
    if (!voa) bsum_a = 0.f;
    if (!vob) bsum_b = 0.f;
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

// The same for a job whose O and I are multiples of 64 and whose rows are 16-byte aligned (x, dy and their row strides),
// which is every projection of the encoder layers.  The four wavefronts of the workgroup share ONE 64x64 block of dW
// (64 ty, 64 tx) and split the rows of the slice; each holds the block as sixteen accumulators, and a lane reads FOUR
// consecutive columns of a row at once.  They feed four different accumulator tiles: tile jo of dY holds the columns
// o0 + 4 m + jo (m = 0..15 the tile's row index), tile ji of X the columns i0 + 4 n + ji, so that accumulator (jo, ji) is
// the block's elements (4 m + jo, 4 n + ji) -- a renumbering of the block's rows and columns that is undone where the
// four blocks are added up in LDS.  A step of four rows is 2 loads of 256 contiguous bytes per row for 16 matrix
// instructions, against 4 loads of 64 bytes for 4 in wgrad_block, where the wavefronts spent 60 % of their time waiting
// for loads; and the block reaches memory as one float atomic per element and workgroup, whole rows at a time.
constexpr int WG_LDS_ROW = 68;    // floats per row of the block in LDS (16-byte rows, spread over the banks)
__device__ __forceinline__ void wgrad_block_wide(const float* __restrict__ x, const float* __restrict__ dy, int N, int I,
                                                 int O, int ldx, int ldy, int rows_per_slice, int tx, int ty, int slice,
                                                 float* dW, float* db, float* block /* LDS [64][WG_LDS_ROW] */) {
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
    const int o0 = ty * 64, i0 = tx * 64;
    // this wavefront's rows of the slice: a quarter, in whole steps of four rows
    const int s0 = slice * rows_per_slice, s1 = min(N, s0 + rows_per_slice);
    const int quarter = (((s1 - s0 + 3) >> 2) + 3) & ~3;
    const int r0 = min(s1, s0 + w * quarter), r1 = min(s1, r0 + quarter);
    const int col = lane & 15, kk = lane >> 4;
    constexpr int UN = 2;                                 // steps of four rows per chunk
    const char* by = reinterpret_cast<const char*>(dy + (size_t)r0 * ldy + o0 + 4 * col);      // the chunk's first row
    const char* bx = reinterpret_cast<const char*>(x + (size_t)r0 * ldx + i0 + 4 * col);
    uint32_t oy[UN], ox[UN];                              // byte offsets of the lane's rows within a chunk
#pragma unroll
    for (int u = 0; u < UN; u++) {
        oy[u] = 4u * (uint32_t)(kk + 4 * u) * (uint32_t)ldy;
        ox[u] = 4u * (uint32_t)(kk + 4 * u) * (uint32_t)ldx;
    }
    const size_t sy = (size_t)4 * UN * 4 * ldy, sx = (size_t)4 * UN * 4 * ldx;   // bytes per chunk
    v4f_l acc[4][4];
#pragma unroll
    for (int a = 0; a < 4; a++)
#pragma unroll
        for (int c = 0; c < 4; c++) acc[a][c] = v4f_l{0.f, 0.f, 0.f, 0.f};
    v4f_l bsum = {0.f, 0.f, 0.f, 0.f};
    auto ld4 = [](const char* base, uint32_t off) { return *reinterpret_cast<const v4f_l*>(base + off); };
    auto products = [&](const v4f_l (&y4)[UN], const v4f_l (&x4)[UN]) {
#pragma unroll
        for (int u = 0; u < UN; u++) {
#pragma unroll
            for (int a = 0; a < 4; a++)
#pragma unroll
                for (int c = 0; c < 4; c++)
                    acc[a][c] = __builtin_amdgcn_mfma_f32_16x16x4f32(y4[u][a], x4[u][c], acc[a][c], 0, 0, 0);
            bsum += y4[u];
        }
    };
    const int nfull = (r1 - r0) / (4 * UN);
    if (nfull > 0) {
        v4f_l y4[UN], x4[UN];
#pragma unroll
        for (int u = 0; u < UN; u++) { y4[u] = ld4(by, oy[u]); x4[u] = ld4(bx, ox[u]); }
        for (int c = 1; c < nfull; c++) {
            by += sy; bx += sx;
            v4f_l ny[UN], nx[UN];
#pragma unroll
            for (int u = 0; u < UN; u++) { ny[u] = ld4(by, oy[u]); nx[u] = ld4(bx, ox[u]); }
            products(y4, x4);
#pragma unroll
            for (int u = 0; u < UN; u++) { y4[u] = ny[u]; x4[u] = nx[u]; }
        }
        products(y4, x4);
        by += sy; bx += sx;
    }
    const int rt = r0 + 4 * UN * nfull;                   // the rows left: fewer than a chunk
    if (rt < r1) {
        v4f_l y4[UN], x4[UN];
#pragma unroll
        for (int u = 0; u < UN; u++) {
            const bool vr = rt + kk + 4 * u < r1;         // a row past the end reads the chunk's first row, dY as zero
            y4[u] = ld4(by, vr ? oy[u] : 0u);
            x4[u] = ld4(bx, vr ? ox[u] : 0u);
            if (!vr) y4[u] = v4f_l{0.f, 0.f, 0.f, 0.f};
        }
        products(y4, x4);
    }
    // accumulator (a, c), component e of lane (kk, col): element (4 (4 kk + e) + a, 4 col + c) of the block.  The four
    // wavefronts add their blocks up in LDS one after the other, 16 bytes per lane and access (LDS float atomics took
    // several times as long as the products).
#pragma unroll 1
    for (int ph = 0; ph < 4; ph++) {
        if (w == ph) {
#pragma unroll
            for (int a = 0; a < 4; a++)
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    v4f_l* const p = reinterpret_cast<v4f_l*>(block + (4 * (4 * kk + e) + a) * WG_LDS_ROW + 4 * col);
                    v4f_l v = {acc[a][0][e], acc[a][1][e], acc[a][2][e], acc[a][3][e]};
                    if (ph > 0) v += *p;
                    *p = v;
                }
        }
        __syncthreads();
    }
    if (db && tx == 0 && r1 > r0) {                       // one column of blocks sums dY over its rows
#pragma unroll
        for (int a = 0; a < 4; a++) {
            const float sum = rows_sum(bsum[a]);
            if (kk == 0) atomicAdd(db + o0 + 4 * col + a, sum);
        }
    }
    for (int idx = threadIdx.x; idx < 64 * 64; idx += 256) {
        const int m = idx >> 6, n = idx & 63;
        atomicAdd(dW + (size_t)(o0 + m) * I + i0 + n, block[m * WG_LDS_ROW + n]);
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
    int wide;         // wgrad_block_wide instead of wgrad_block
};
struct WgradJobs { WgradJob job[WGRAD_MAX_JOBS]; int njobs, blocks; };

// The grid is a multiple of 8 workgroups.  Consecutive workgroups go to the 8 dies of the chip in turn, each with an
// L2 of its own; the workgroups that read the same rows of x and dy -- the tiles of one slice of one job, consecutive in
// the numbering of the job table -- are therefore renumbered so that they share a die (numbered in turn, every die
// fetched nearly every row: 78 % of the L2 requests missed).
// (at most 128 registers: four workgroups a compute unit, which is what the host sizes the slices for)
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(4, 4))) void linear_wgrad_batch_kernel(const WgradJobs T) {
    const int per_die = (int)gridDim.x >> 3;
    const int block = ((int)blockIdx.x & 7) * per_die + ((int)blockIdx.x >> 3);
    if (block >= T.blocks) return;
    int j = 0;
    for (int t = 1; t < T.njobs; t++)
        if (block >= T.job[t].block0) j = t;
    const WgradJob& J = T.job[j];
    const int b = block - J.block0;
    const int tiles = J.bx * J.by;
    const int slice = b / tiles, tile = b - slice * tiles;
    __shared__ __attribute__((aligned(16))) float lds_block[64 * WG_LDS_ROW];
    if (J.wide)
        wgrad_block_wide(J.x, J.dy, J.N, J.I, J.O, J.ldx, J.ldy, J.rows_per_slice, tile % J.bx, tile / J.bx, slice, J.dW, J.db,
                         lds_block);
    else
        wgrad_block(J.x, J.dy, J.N, J.I, J.O, J.ldx, J.ldy, J.rows_per_slice, tile % J.bx, tile / J.bx, slice, J.dW, J.db);
}

__global__ __launch_bounds__(256) void zero2_kernel(float* a, int na, float* b, int nb) {
    const int idx = blockIdx.x * blockDim.x + threadIdx.x;
    if (idx < na) a[idx] = 0.0f;
    if (b && idx < nb) b[idx] = 0.0f;
}

}  // namespace cfh
