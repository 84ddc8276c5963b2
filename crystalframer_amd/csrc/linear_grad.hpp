// Weight and bias gradients of y = x W^T + b for the projections around the attention
// (N rows = atoms, a few hundred columns):  dW (O,I) = dY^T X,  db (O) = sum over rows of dY.
// The library GEMM the framework would call picks a 32x32 tile without splitting the long
// dimension for these shapes (16 workgroups for a 128x128 output, 19 us) and the bias gradient is
// a second launch; here the N rows are split over gridDim.z slices so that a launch fills the chip,
// each wavefront owns a 32x32 block of dW as four v_mfma_f32_16x16x4 accumulators.  The slices of a 64x64 tile are
// combined either with float atomics into the outputs (the sum order, and the last bits, then differ from run to
// run) or, when the caller provides scratch, in a fixed order: every workgroup stores its tile, and a second small
// kernel adds the stored tiles up slice by slice (bit-reproducible).
#pragma once
#include "device_common.hpp"

namespace cfh {

typedef float v4f_l __attribute__((ext_vector_type(4)));

// One workgroup's share: 256 threads = 4 wavefronts, wavefront w owns the 32x32 block
// (64 ty + 32 (w/2), 64 tx + 32 (w%2)) of dW and the rows [slice rows_per_slice, ...) of x and dy
// (row strides ldx, ldy: dy may be a column slice of a wider matrix).  dW == nullptr: only db is
// computed (x is not read; I = 1).
constexpr int WG_LDS_ROW = 68;    // floats per row of the workgroup's 64x64 tile in LDS (16-byte rows, spread over the banks)
// Leaves the workgroup's share of the tile (64 ty, 64 tx) in `block` and the column sums of its dY rows in `colsum`
// (both cleared by the caller).
__device__ __forceinline__ void wgrad_block(const float* __restrict__ x, const float* __restrict__ dy, int N, int I,
                                            int O, int ldx, int ldy, int rows_per_slice, int tx, int ty, int slice,
                                            bool has_dw, float* block, float* colsum) {
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
    const bool has_w = has_dw;                            // no dW: the column sums of dY alone
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
    // accumulator component c of lane (kk, col): row 4 kk + c of the 16x16 block, column col: into the workgroup's
    // 64x64 tile in LDS (rows / columns past the edges of dW hold copies that the output step leaves out)
    const int ro = 32 * (w >> 1), co = 32 * (w & 1);
#pragma unroll
    for (int c = 0; c < 4; c++) {
        const int oo = ro + 4 * kk + c;
        block[oo * WG_LDS_ROW + co + col] = acc00[c];
        block[oo * WG_LDS_ROW + co + 16 + col] = acc01[c];
        block[(oo + 16) * WG_LDS_ROW + co + col] = acc10[c];
        block[(oo + 16) * WG_LDS_ROW + co + 16 + col] = acc11[c];
    }
    if ((w & 1) == 0) {                                   // one column of wavefronts sums dY over its rows
        bsum_a = rows_sum(bsum_a);
        bsum_b = rows_sum(bsum_b);
        if (kk == 0) { colsum[ro + col] = bsum_a; colsum[ro + 16 + col] = bsum_b; }
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
__device__ __forceinline__ void wgrad_block_wide(const float* __restrict__ x, const float* __restrict__ dy, int N, int I,
                                                 int O, int ldx, int ldy, int rows_per_slice, int tx, int ty, int slice,
                                                 float* block /* LDS [64][WG_LDS_ROW] */, float* colsum4 /* LDS [4][64] */) {
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
    // this wavefront's column sums of dY (tile columns 4 col + a), added up over the wavefronts by the caller
#pragma unroll
    for (int a = 0; a < 4; a++) {
        const float sum = rows_sum(bsum[a]);
        if (kk == 0) colsum4[w * 64 + 4 * col + a] = sum;
    }
}

// Scratch of a launch whose sums run in a fixed order (null: float atomics into the outputs): the tiles as the
// workgroups computed them, WG_PART floats each, in the order of the workgroups' numbers.
struct WgradScratch {
    float* partials;
};
constexpr int WG_PART = 64 * 64 + 64;      // floats a workgroup stores: its tile and its 64 column sums

// Output of one workgroup's tile: `block` (64x64 in LDS) and `colsum` (64) are its share of tile (ty, tx) of the job,
// slice `slice` of `slices`; `wg` its number in the launch.
__device__ __forceinline__ void wgrad_output(const float* block, const float* colsum, float* dW, float* db, int O, int I,
                                             int tx, int ty, int slices, int wg, const WgradScratch& S) {
    const int o0 = ty * 64, i0 = tx * 64;
    const bool bias = db != nullptr && tx == 0;
    if (S.partials == nullptr) {                          // float atomics, any order
        if (dW)
            for (int idx = threadIdx.x; idx < 64 * 64; idx += 256) {
                const int m = idx >> 6, n = idx & 63;
                if (o0 + m < O && i0 + n < I) atomicAdd(dW + (size_t)(o0 + m) * I + i0 + n, block[m * WG_LDS_ROW + n]);
            }
        if (bias && threadIdx.x < 64 && o0 + (int)threadIdx.x < O) atomicAdd(db + o0 + threadIdx.x, colsum[threadIdx.x]);
        return;
    }
    if (slices == 1) {                                    // the only writer of this tile
        if (dW)
            for (int idx = threadIdx.x; idx < 64 * 64; idx += 256) {
                const int m = idx >> 6, n = idx & 63;
                if (o0 + m < O && i0 + n < I) dW[(size_t)(o0 + m) * I + i0 + n] += block[m * WG_LDS_ROW + n];
            }
        if (bias && threadIdx.x < 64 && o0 + (int)threadIdx.x < O) db[o0 + threadIdx.x] += colsum[threadIdx.x];
        return;
    }
    // stored for linear_wgrad_sum_kernel: the 16-byte pieces q = threadIdx.x + 256 j (row q / 16, columns 4 (q % 16) ...)
    float* const part = S.partials + (size_t)wg * WG_PART;
    if (dW) {
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const int q = threadIdx.x + 256 * j;
            *reinterpret_cast<v4f_l*>(part + 4 * q) = *reinterpret_cast<const v4f_l*>(block + (q >> 4) * WG_LDS_ROW + 4 * (q & 15));
        }
    }
    if (bias && threadIdx.x < 64) part[64 * 64 + threadIdx.x] = colsum[threadIdx.x];
}

// One workgroup's tile from the products to the outputs.  `wide`: the variant with 16-byte loads.
__device__ __forceinline__ void wgrad_tile(const float* __restrict__ x, const float* __restrict__ dy, int N, int I, int O,
                                           int ldx, int ldy, int rows_per_slice, int tx, int ty, int slice, int slices,
                                           float* dW, float* db, bool wide, int wg, const WgradScratch& S) {
    __shared__ __attribute__((aligned(16))) float lds_block[64 * WG_LDS_ROW];
    __shared__ float lds_colsum[4 * 64];
    if (wide) {
        wgrad_block_wide(x, dy, N, I, O, ldx, ldy, rows_per_slice, tx, ty, slice, lds_block, lds_colsum);
        __syncthreads();
        if (threadIdx.x < 64)
            lds_colsum[threadIdx.x] = (lds_colsum[threadIdx.x] + lds_colsum[64 + threadIdx.x]) +
                                      (lds_colsum[128 + threadIdx.x] + lds_colsum[192 + threadIdx.x]);
    } else {
        for (int idx = threadIdx.x; idx < 64 * WG_LDS_ROW; idx += 256) lds_block[idx] = 0.0f;
        if (threadIdx.x < 64) lds_colsum[threadIdx.x] = 0.0f;
        __syncthreads();
        wgrad_block(x, dy, N, I, O, ldx, ldy, rows_per_slice, tx, ty, slice, dW != nullptr, lds_block, lds_colsum);
    }
    __syncthreads();
    wgrad_output(lds_block, lds_colsum, dW, db, O, I, tx, ty, slices, wg, S);
}

// grid: (ceil(I/64), ceil(O/64), slices), block: 256 threads; float atomics into the cleared outputs
__global__ __launch_bounds__(256) void linear_wgrad_kernel(const float* __restrict__ x, const float* __restrict__ dy,
                                                           int N, int I, int O, int rows_per_slice,
                                                           float* dW, float* db) {
    const WgradScratch none{nullptr};
    wgrad_tile(x, dy, N, I, O, I, O, rows_per_slice, blockIdx.x, blockIdx.y, blockIdx.z, (int)gridDim.z, dW, db, false, 0,
               none);
}

// Several layers' gradients in one launch: the jobs travel in the kernel arguments, workgroup b
// belongs to the job with block0 <= b < block0 + bx by slices.
constexpr int WGRAD_MAX_JOBS = 32;
struct WgradJob {
    const float* x; const float* dy; float* dW; float* db;
    int N, I, O, ldx, ldy;
    int block0, bx, by, rows_per_slice;
    int slices;       // of the rows
    int tile0;        // number of the job's first tile among the tiles of the launch that several slices share
    int wide;         // wgrad_block_wide instead of wgrad_block
};
struct WgradJobs { WgradJob job[WGRAD_MAX_JOBS]; int njobs, blocks, split_tiles; WgradScratch scratch; };

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
    wgrad_tile(J.x, J.dy, J.N, J.I, J.O, J.ldx, J.ldy, J.rows_per_slice, tile % J.bx, tile / J.bx, slice, J.slices, J.dW, J.db,
               J.wide != 0, block, T.scratch);
}

// Second step of a launch with scratch: the stored tiles of every tile that several slices share, added up in the
// order of the slices and added to the outputs.  grid: 4 workgroups per such tile (16 rows of the tile each, one
// 16-byte piece per thread), block: 256 threads.  The loads of eight slices are in flight together.
__global__ __launch_bounds__(256) void linear_wgrad_sum_kernel(const WgradJobs T) {
    const int t = (int)blockIdx.x >> 2, quarter = (int)blockIdx.x & 3;
    if (t >= T.split_tiles) return;
    int j = -1;
    for (int n = 0; n < T.njobs; n++)
        if (T.job[n].slices > 1 && t >= T.job[n].tile0) j = n;
    if (j < 0) return;
    const WgradJob& J = T.job[j];
    const int tile = t - J.tile0, tiles = J.bx * J.by;
    if (tile >= tiles) return;
    const int tx = tile % J.bx, ty = tile / J.bx;
    const int o0 = ty * 64, i0 = tx * 64;
    const float* const first = T.scratch.partials + (size_t)(J.block0 + tile) * WG_PART;
    const size_t step = (size_t)tiles * WG_PART;          // from one slice of the tile to the next
    const int slices = J.slices;
    // (the column sums ride along with the tile's loads: a loop of their own, one slice after the other, took as long
    // as the tile)
    const int q = 256 * quarter + (int)threadIdx.x;
    const bool has_w = J.dW != nullptr;
    const bool do_bias = J.db && tx == 0 && quarter == 0 && threadIdx.x < 64 && o0 + (int)threadIdx.x < J.O;
    const int m = q >> 4, n = 4 * (q & 15);
    const bool row_ok = has_w && o0 + m < J.O;
    float* const dst = has_w ? J.dW + (size_t)(o0 + min(m, J.O - 1 - o0)) * J.I + i0 + n : nullptr;
    const bool vec = row_ok && (J.I & 3) == 0 && (reinterpret_cast<uintptr_t>(J.dW) & 15) == 0 && i0 + n + 3 < J.I;
    // what the outputs hold is asked for before the stored tiles, not after them
    v4f_l sum = {0.f, 0.f, 0.f, 0.f};
    if (vec) sum = *reinterpret_cast<const v4f_l*>(dst);
    float bsum = do_bias ? J.db[o0 + threadIdx.x] : 0.0f;
    v4f_l add = {0.f, 0.f, 0.f, 0.f};
    float badd = 0.0f;
    for (int sl = 0; sl < slices; sl += 8) {
        v4f_l t[8];
        float tb[8];
#pragma unroll
        for (int u = 0; u < 8; u++) {                     // past the last slice: the batch's first slice again, not added
            const float* const part = first + (size_t)(sl + u < slices ? sl + u : sl) * step;
            t[u] = has_w ? *reinterpret_cast<const v4f_l*>(part + 4 * q) : v4f_l{0.f, 0.f, 0.f, 0.f};
            tb[u] = part[64 * 64 + (threadIdx.x & 63)];
        }
#pragma unroll
        for (int u = 0; u < 8; u++)
            if (sl + u < slices) { add += t[u]; badd += tb[u]; }
    }
    if (vec) {
        *reinterpret_cast<v4f_l*>(dst) = sum + add;
    } else if (row_ok) {
#pragma unroll
        for (int e = 0; e < 4; e++)
            if (i0 + n + e < J.I) dst[e] += add[e];
    }
    if (do_bias) J.db[o0 + threadIdx.x] = bsum + badd;
}

__global__ __launch_bounds__(256) void zero2_kernel(float* a, int na, float* b, int nb) {
    const int idx = blockIdx.x * blockDim.x + threadIdx.x;
    if (idx < na) a[idx] = 0.0f;
    if (b && idx < nb) b[idx] = 0.0f;
}

}  // namespace cfh
