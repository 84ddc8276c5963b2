// The projections between the attention cores of two consecutive encoder layers, which act on every atom
// (row) separately, in one launch:
//     x1  = x_res + attn Wo^T + bo              (output projection of the attention + residual)
//     h   = relu(x1 W1^T + b1)                  (feed-forward, first half)
//     x2  = x1 + h W2^T + b2                    (second half + residual: the layer's output)
//     qkv = x2 Wqkv^T + bqkv                    (stacked input projection of the NEXT layer, optional)
//     qs, k, v, a = split / scaled query / Gaussian coefficient of qkv (see attention_inputs.hpp)
// The reference runs them as separate framework calls (models/indexed_lattice_multi_head_attention_cuda.py:
// 399-409 and the out_proj behind :734, models/indexed_latticeformer_encoder.py:606-648 with post-norm
// switched off), here 4 library GEMMs, 2 additions and the attention-input launch per layer, each a
// few microseconds of work behind a launch.  A workgroup takes 16 rows -- the M of v_mfma_f32_16x16x4 --
// through the whole chain with the activations in LDS; its wavefronts share the output columns of a
// stage, 16 at a time, and stream the weights from the L2.  Every intermediate is also written out:
// the backward pass needs all of them.
#pragma once
#include "device_common.hpp"

namespace cfh {

typedef float v4f_b2 __attribute__((ext_vector_type(4)));

constexpr int BR_ROWS = 16;       // rows (atoms) per workgroup
constexpr int BR_WAVES = 8;
constexpr int BR_PAD = 4;         // floats of padding per LDS row
constexpr int BR_STAGE_FLOATS = 64 * (32 + BR_PAD);    // per wavefront: the weights of one batch of products (forward)

struct BridgeArgs {
    const float* attn; const float* xres;         // (N, D)
    const float* Wo; const float* bo;             // (D, D), (D)        biases may be null
    const float* W1; const float* b1;             // (F, D), (F)
    const float* W2; const float* b2;             // (D, F), (D)
    const float* Wq; const float* bq;             // (3 D, D), (3 D); Wq null: the chain ends with x2
    const float* lattice_w; const float* gauss;   // (D); device {scale, shift} or null
    float* x1; float* h; float* x2; float* qkv;   // (N, D), (N, F), (N, D), (N, 3 D)
    float* qs; float* k; float* v; float* a;      // (N, D) x 3, (N, H)
    int N, D, F, H;
    float c1, lb, c2, q_scale;
};

// out[m][n] = act(sum_k in[m][k] W[n][k] + b[n] + res[m][n]) for the 16 rows of the block and the T column
// tiles (of 16) wave, wave + 4, ... from tile t0 on.  in: LDS [16][K + BR_PAD]; out_lds: LDS [16][O + BR_PAD]
// or null; out_g / res: global rows r0.., row stride O; res_lds: LDS [16][O + BR_PAD] or null.  U: steps of 16
// along K whose loads are in flight.
template <bool RELU, int T, int U>
__device__ __forceinline__ void bridge_tiles(const float* in, int K, const float* __restrict__ W,
                                             const float* __restrict__ b, int O, const float* __restrict__ res,
                                             const float* res_lds, int r0, int nrows, float* out_lds,
                                             float* __restrict__ out_g, int t0, float* stage) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int col = lane & 15, kk = lane >> 4;
    const int ldin = K + BR_PAD, ldout = O + BR_PAD;
    const float* const arow = in + col * ldin + 4 * kk;
    // The weights of the T tiles for 16 U steps of k: (16 T rows) x (16 U floats), T U float4 per lane.  A lane of the
    // matrix operand needs four consecutive k of ITS row, and the 16 lanes of a quarter wavefront hold 16 different
    // rows: read straight from memory that is 64 cache lines per load instruction, which the vector cache takes
    // one per cycle -- twice the time of the products.  So the wavefront reads whole row pieces (16 U floats of a row
    // by 4 U consecutive lanes) and turns them in a piece of LDS of its own.
    constexpr int CH = 4 * U;                     // float4 per row piece
    constexpr int LDS_ROW = 16 * U + BR_PAD;      // floats per staged row (the padding spreads the rows over the banks)
    const float* wsrc[T * U];
    int wdst[T * U];
#pragma unroll
    for (int i = 0; i < T * U; i++) {
        const int q = i * 64 + lane, row = q / CH, ch = q % CH;
        const int tt = row >> 4, j = row & 15;
        wsrc[i] = W + (size_t)(16 * (t0 + wave + BR_WAVES * tt) + j) * K + 4 * ch;
        wdst[i] = row * LDS_ROW + 4 * ch;
    }
    const float* const srow = stage + col * LDS_ROW + 4 * kk;       // tile tt: + 16 tt LDS_ROW
    v4f_b2 acc[T];
#pragma unroll
    for (int tt = 0; tt < T; tt++) acc[tt] = v4f_b2{0.f, 0.f, 0.f, 0.f};
    constexpr int STEP = 16 * U;
    v4f_b2 g4[T * U];
#pragma unroll
    for (int i = 0; i < T * U; i++) g4[i] = *reinterpret_cast<const v4f_b2*>(wsrc[i]);
    // bias and residual of the lane's outputs: asked for now, used behind the products
    float add[T][4];
#pragma unroll
    for (int tt = 0; tt < T; tt++) {
        const int n = 16 * (t0 + wave + BR_WAVES * tt) + col;
        const float bias = b ? b[n] : 0.f;
#pragma unroll
        for (int c = 0; c < 4; c++) {
            const int m = 4 * kk + c;
            add[tt][c] = bias + (res && m < nrows ? res[(size_t)(r0 + m) * O + n] : 0.f);
        }
    }
    for (int k0 = 0; k0 < K; k0 += STEP) {
        wave_sync();                               // the products of the step before have read the stage
#pragma unroll
        for (int i = 0; i < T * U; i++) *reinterpret_cast<v4f_b2*>(stage + wdst[i]) = g4[i];
        {   // the next batch is asked for before the products of this one (the last one once more at the end: no
            // branch around the loads).  Asking two steps ahead gains nothing: a compute unit takes about 20 bytes a
            // cycle from the L2 however many loads are in flight, and the 768 KB of weights that every workgroup
            // streams make that the bound of the kernel (18 us), above the 10 us of its matrix instructions.
            const int kn = k0 + STEP < K ? k0 + STEP : k0;
#pragma unroll
            for (int i = 0; i < T * U; i++) g4[i] = *reinterpret_cast<const v4f_b2*>(wsrc[i] + kn);
        }
        wave_sync();
        float4 a4[U], w4[U][T];
#pragma unroll
        for (int u = 0; u < U; u++) {
            a4[u] = *reinterpret_cast<const float4*>(arow + k0 + 16 * u);
#pragma unroll
            for (int tt = 0; tt < T; tt++)
                w4[u][tt] = *reinterpret_cast<const float4*>(srow + 16 * tt * LDS_ROW + 16 * u);
        }
#pragma unroll
        for (int u = 0; u < U; u++)
#pragma unroll
            for (int tt = 0; tt < T; tt++) {
                acc[tt] = __builtin_amdgcn_mfma_f32_16x16x4f32(a4[u].x, w4[u][tt].x, acc[tt], 0, 0, 0);
                acc[tt] = __builtin_amdgcn_mfma_f32_16x16x4f32(a4[u].y, w4[u][tt].y, acc[tt], 0, 0, 0);
                acc[tt] = __builtin_amdgcn_mfma_f32_16x16x4f32(a4[u].z, w4[u][tt].z, acc[tt], 0, 0, 0);
                acc[tt] = __builtin_amdgcn_mfma_f32_16x16x4f32(a4[u].w, w4[u][tt].w, acc[tt], 0, 0, 0);
            }
    }
#pragma unroll
    for (int tt = 0; tt < T; tt++) {
        const int n = 16 * (t0 + wave + BR_WAVES * tt) + col;
#pragma unroll
        for (int c = 0; c < 4; c++) {
            const int m = 4 * kk + c;
            float val = acc[tt][c] + add[tt][c];
            if (res_lds) val += res_lds[m * ldout + n];
            if (RELU) val = fmaxf(val, 0.f);
            if (out_lds) out_lds[m * ldout + n] = val;
            if (m < nrows) out_g[(size_t)(r0 + m) * O + n] = val;
        }
    }
}

// All O columns (O a multiple of 64: whole tiles for each of the four wavefronts; K a multiple of 64).
template <bool RELU>
__device__ __forceinline__ void bridge_stage(const float* in, int K, const float* __restrict__ W,
                                             const float* __restrict__ b, int O, const float* __restrict__ res,
                                             const float* res_lds, int r0, int nrows, float* out_lds,
                                             float* __restrict__ out_g, float* stage) {
    int t0 = 0;
    int left = O / (16 * BR_WAVES);     // tiles per wavefront still to do
    while (left >= 4) { bridge_tiles<RELU, 4, 2>(in, K, W, b, O, res, res_lds, r0, nrows, out_lds, out_g, t0, stage); t0 += 4 * BR_WAVES; left -= 4; }
    if (left >= 2) { bridge_tiles<RELU, 2, 4>(in, K, W, b, O, res, res_lds, r0, nrows, out_lds, out_g, t0, stage); t0 += 2 * BR_WAVES; left -= 2; }
    if (left >= 1) { bridge_tiles<RELU, 1, 8>(in, K, W, b, O, res, res_lds, r0, nrows, out_lds, out_g, t0, stage); }
}

// grid: ceil(N / 16) workgroups of 512 threads; dynamic LDS: 16 (2 (D + 4) + max(F, 3 D) + 4) floats and
// BR_STAGE_FLOATS per wavefront.
// D, F multiples of 128; D = 16 H.
__global__ __launch_bounds__(64 * BR_WAVES) void layer_bridge_fwd_kernel(const BridgeArgs P) {
    extern __shared__ __attribute__((aligned(16))) float bridge_lds[];
    const int D = P.D, F = P.F, Q = 3 * D;
    float* const s_a = bridge_lds;                            // [16][D+4]  attention output, later x2
    float* const s_b = s_a + BR_ROWS * (D + BR_PAD);          // [16][D+4]  x1
    float* const s_c = s_b + BR_ROWS * (D + BR_PAD);          // [16][F+4]  h, later [16][3D+4] qkv
    float* const stage = s_c + BR_ROWS * ((F > Q ? F : Q) + BR_PAD) + (threadIdx.x >> 6) * BR_STAGE_FLOATS;
    const int r0 = blockIdx.x * BR_ROWS;
    const int nrows = min(BR_ROWS, P.N - r0);
    for (int idx = threadIdx.x * 4; idx < BR_ROWS * D; idx += 64 * BR_WAVES * 4) {
        const int m = idx / D, c = idx - m * D;
        float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
        if (m < nrows) v = *reinterpret_cast<const float4*>(P.attn + (size_t)(r0 + m) * D + c);
        *reinterpret_cast<float4*>(s_a + m * (D + BR_PAD) + c) = v;
    }
    __syncthreads();
    bridge_stage<false>(s_a, D, P.Wo, P.bo, D, P.xres, nullptr, r0, nrows, s_b, P.x1, stage);
    __syncthreads();
    bridge_stage<true>(s_b, D, P.W1, P.b1, F, nullptr, nullptr, r0, nrows, s_c, P.h, stage);
    __syncthreads();
    bridge_stage<false>(s_c, F, P.W2, P.b2, D, nullptr, s_b, r0, nrows, s_a, P.x2, stage);
    if (!P.Wq) return;
    __syncthreads();
    bridge_stage<false>(s_a, D, P.Wq, P.bq, Q, nullptr, nullptr, r0, nrows, s_c, P.qkv, stage);
    __syncthreads();
    // split of qkv, query scaling
    const int ldq = Q + BR_PAD;
    for (int idx = threadIdx.x * 4; idx < BR_ROWS * Q; idx += 64 * BR_WAVES * 4) {
        const int m = idx / Q, c = idx - m * Q;
        if (m >= nrows) break;
        float4 val = *reinterpret_cast<const float4*>(s_c + m * ldq + c);
        const int part = c / D, cc = c - part * D;
        float* dst = part == 0 ? P.qs : (part == 1 ? P.k : P.v);
        if (part == 0) { val.x *= P.q_scale; val.y *= P.q_scale; val.z *= P.q_scale; val.w *= P.q_scale; }
        *reinterpret_cast<float4*>(dst + (size_t)(r0 + m) * D + cc) = val;
    }
    // Gaussian coefficient of every (row, head)
    if ((int)threadIdx.x < BR_ROWS * P.H) {
        const int m = threadIdx.x / P.H, hh = threadIdx.x - m * P.H;
        if (m < nrows) {
            float alpha = 0.0f;
#pragma unroll
            for (int d = 0; d < DH; d++) alpha = fmaf(s_c[m * ldq + hh * DH + d], P.lattice_w[hh * DH + d], alpha);
            if (P.gauss) alpha = (alpha + P.gauss[1]) * P.gauss[0];
            const float u = alpha * P.c1;
            const float e = u > 0.0f ? u : expm1f(u);
            P.a[(size_t)(r0 + m) * P.H + hh] = ((1.0f - P.lb) * e + 1.0f) * P.c2;
        }
    }
}


// ---- backward: the input gradients of the same chain ------------------------------------------------
//     g2 = g_x2 + gqkv Wqkv;   gh = (g2 W2) [h > 0];   g1 = g2 + gh W1;   g_attn = g1 Wo
// (weights as stored, (out, in) row-major, so these are products with W itself: row k of W is
// contiguous along the output column n).  Every intermediate is written out: the weight-gradient
// launch at the end of the backward pass multiplies them with the saved activations.
struct BridgeBwdArgs {
    const float* g_x2;            // (N, D) or null (zero)
    const float* gqkv;            // (N, 3 D) or null: no next layer, g2 = g_x2 (g2 is then not written)
    const float* h;               // (N, F) forward activations (the rectifier's mask)
    const float* Wq; const float* W2; const float* W1; const float* Wo;     // (3D, D), (D, F), (F, D), (D, D)
    float* g2; float* gh; float* g1; float* g_attn;                         // (N, D), (N, F), (N, D), (N, D)
    int N, D, F;
    // optional: gqkv is not given but made here from the gradients of the attention inputs (the backward of
    // attention_inputs.hpp for the 16 rows of the block), written to gqkv_out for the weight-gradient launch
    const float* ai_qkv;          // (N, 3 D) forward projection output; null: gqkv above is used
    const float* ai_w; const float* ai_gauss;
    const float* ai_gqs; const float* ai_gk; const float* ai_gv; const float* ai_ga;    // each may be null (zero)
    float* gqkv_out;              // (N, 3 D)
    float* gw_partial;            // (blocks, D): this block's sum over its rows of the lattice-weight gradient
    int H;
    float c1, lb, c2, q_scale;
};

// Partial products of one stage: out[m][n] += sum over this wavefront's share of k of in[m][k] W[k][n].
// The 8 wavefronts split the work as (group of 64 output columns) x (slice of K); a lane's float4 of W holds
// the columns n0 + 4 col .. + 3 of one row k, which feed four accumulators (column n0 + 4 col + tt), and
// the four steps of a chunk of 16 k take k = k0 + 4 kk + t (the float4 of the LDS operand holds the same four).
// part: LDS [slices][16][O + BR_PAD].
__device__ __forceinline__ void bridge_bwd_products(const float* in, int K, const float* __restrict__ W, int O,
                                                    float* part) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int col = lane & 15, kk = lane >> 4;
    const int ngroups = O >> 6;
    const int slices = ngroups >= BR_WAVES ? 1 : BR_WAVES / ngroups;
    const int ldin = K + BR_PAD, ldp = O + BR_PAD;
    const int klen = K / slices;                      // a multiple of 32: K is a multiple of 128, slices <= 4
    for (int unit = wave; unit < ngroups * slices; unit += BR_WAVES) {
        const int grp = unit / slices, sl = unit - grp * slices;
        const int n0 = 64 * grp, kbeg = sl * klen;
        v4f_b2 acc[4];
#pragma unroll
        for (int tt = 0; tt < 4; tt++) acc[tt] = v4f_b2{0.f, 0.f, 0.f, 0.f};
        const float* const arow = in + col * ldin + kbeg + 4 * kk;
        const float* const wbase = W + (size_t)(kbeg + 4 * kk) * O + n0 + 4 * col;
        for (int k0 = 0; k0 < klen; k0 += 32) {
            float4 a4[2], w4[2][4];
#pragma unroll
            for (int u = 0; u < 2; u++) {
                a4[u] = *reinterpret_cast<const float4*>(arow + k0 + 16 * u);
#pragma unroll
                for (int t = 0; t < 4; t++)
                    w4[u][t] = *reinterpret_cast<const float4*>(wbase + (size_t)(k0 + 16 * u + t) * O);
            }
#pragma unroll
            for (int u = 0; u < 2; u++) {
                const float av[4] = {a4[u].x, a4[u].y, a4[u].z, a4[u].w};
#pragma unroll
                for (int t = 0; t < 4; t++) {
                    acc[0] = __builtin_amdgcn_mfma_f32_16x16x4f32(av[t], w4[u][t].x, acc[0], 0, 0, 0);
                    acc[1] = __builtin_amdgcn_mfma_f32_16x16x4f32(av[t], w4[u][t].y, acc[1], 0, 0, 0);
                    acc[2] = __builtin_amdgcn_mfma_f32_16x16x4f32(av[t], w4[u][t].z, acc[2], 0, 0, 0);
                    acc[3] = __builtin_amdgcn_mfma_f32_16x16x4f32(av[t], w4[u][t].w, acc[3], 0, 0, 0);
                }
            }
        }
        float* const dst = part + (size_t)sl * BR_ROWS * ldp + n0 + 4 * col;
#pragma unroll
        for (int c = 0; c < 4; c++)
            *reinterpret_cast<float4*>(dst + (4 * kk + c) * ldp) = make_float4(acc[0][c], acc[1][c], acc[2][c], acc[3][c]);
    }
}

// out[m][n] = sum over the slices of part + add (global rows r0.., or LDS, or nothing), times [mask > 0]
// when a mask is given; to LDS (optional) and to global memory.
__device__ __forceinline__ void bridge_bwd_finish(const float* part, int O, const float* __restrict__ add_g,
                                                  const float* add_lds, const float* __restrict__ mask_g, int r0,
                                                  int nrows, float* out_lds, float* __restrict__ out_g) {
    const int ngroups = O >> 6;
    const int slices = ngroups >= BR_WAVES ? 1 : BR_WAVES / ngroups;
    const int ldp = O + BR_PAD;
    for (int idx = threadIdx.x * 4; idx < BR_ROWS * O; idx += 64 * BR_WAVES * 4) {
        const int m = idx / O, n = idx - m * O;
        float4 v = *reinterpret_cast<const float4*>(part + m * ldp + n);
        for (int sl = 1; sl < slices; sl++) {
            const float4 p = *reinterpret_cast<const float4*>(part + ((size_t)sl * BR_ROWS + m) * ldp + n);
            v.x += p.x; v.y += p.y; v.z += p.z; v.w += p.w;
        }
        const bool live = m < nrows;
        const size_t g = (size_t)(r0 + m) * O + n;
        if (add_g && live) {
            const float4 p = *reinterpret_cast<const float4*>(add_g + g);
            v.x += p.x; v.y += p.y; v.z += p.z; v.w += p.w;
        }
        if (add_lds) {
            const float4 p = *reinterpret_cast<const float4*>(add_lds + m * ldp + n);
            v.x += p.x; v.y += p.y; v.z += p.z; v.w += p.w;
        }
        if (mask_g) {
            float4 hm = make_float4(0.f, 0.f, 0.f, 0.f);
            if (live) hm = *reinterpret_cast<const float4*>(mask_g + g);
            v.x = hm.x > 0.f ? v.x : 0.f; v.y = hm.y > 0.f ? v.y : 0.f;
            v.z = hm.z > 0.f ? v.z : 0.f; v.w = hm.w > 0.f ? v.w : 0.f;
        }
        if (out_lds) *reinterpret_cast<float4*>(out_lds + m * ldp + n) = v;
        if (live) *reinterpret_cast<float4*>(out_g + g) = v;
    }
}

// LDS floats the backward kernel needs
__host__ __device__ inline size_t bridge_bwd_lds_floats(int D, int F) {
    const int sl_d = (D >> 6) >= BR_WAVES ? 1 : BR_WAVES / (D >> 6);
    const int sl_f = (F >> 6) >= BR_WAVES ? 1 : BR_WAVES / (F >> 6);
    const size_t part_d = (size_t)sl_d * BR_ROWS * (D + BR_PAD), part_f = (size_t)sl_f * BR_ROWS * (F + BR_PAD);
    return (size_t)BR_ROWS * ((3 * D + BR_PAD) + 2 * (D + BR_PAD) + (F + BR_PAD)) + (part_d > part_f ? part_d : part_f);
}

// grid: ceil(N / 16) workgroups of 512 threads; dynamic LDS: bridge_bwd_lds_floats(D, F) floats.
__global__ __launch_bounds__(64 * BR_WAVES) void layer_bridge_bwd_kernel(const BridgeBwdArgs P) {
    extern __shared__ __attribute__((aligned(16))) float bridge_lds[];
    const int D = P.D, F = P.F, Q = 3 * D;
    float* const s_q = bridge_lds;                            // [16][3D+4] gqkv
    float* const s_g2 = s_q + BR_ROWS * (Q + BR_PAD);         // [16][D+4]
    float* const s_g1 = s_g2 + BR_ROWS * (D + BR_PAD);        // [16][D+4]
    float* const s_gh = s_g1 + BR_ROWS * (D + BR_PAD);        // [16][F+4]
    float* const part = s_gh + BR_ROWS * (F + BR_PAD);
    const int r0 = blockIdx.x * BR_ROWS;
    const int nrows = min(BR_ROWS, P.N - r0);
    if (P.ai_qkv) {
        // gradient of the stacked projection output from the gradients of (qs, k, v, a)
        const int ldd = D + BR_PAD;
        float* const s_qf = s_g1;                 // [16][D+4] the forward query rows (s_g1 is free until later)
        float* const s_ga = part;                 // [16][H]   ga da/dalpha
        for (int idx = threadIdx.x * 4; idx < BR_ROWS * D; idx += 64 * BR_WAVES * 4) {
            const int m = idx / D, c = idx - m * D;
            float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
            if (m < nrows) v = *reinterpret_cast<const float4*>(P.ai_qkv + (size_t)(r0 + m) * Q + c);
            *reinterpret_cast<float4*>(s_qf + m * ldd + c) = v;
        }
        __syncthreads();
        if ((int)threadIdx.x < BR_ROWS * P.H) {
            const int m = threadIdx.x / P.H, hh = threadIdx.x - m * P.H;
            float galpha = 0.0f;
            if (m < nrows && P.ai_ga) {
                float alpha = 0.0f, scale = 1.0f;
#pragma unroll
                for (int d = 0; d < DH; d++) alpha = fmaf(s_qf[m * ldd + hh * DH + d], P.ai_w[hh * DH + d], alpha);
                if (P.ai_gauss) { scale = P.ai_gauss[0]; alpha = (alpha + P.ai_gauss[1]) * scale; }
                const float u = alpha * P.c1;
                const float e = u > 0.0f ? u : expm1f(u);
                const float slope = (u > 0.0f ? 1.0f : e + 1.0f) * P.c1 * scale * (1.0f - P.lb) * P.c2;
                galpha = P.ai_ga[(size_t)(r0 + m) * P.H + hh] * slope;
            }
            s_ga[m * P.H + hh] = galpha;
        }
        __syncthreads();
        for (int idx = threadIdx.x * 4; idx < BR_ROWS * Q; idx += 64 * BR_WAVES * 4) {
            const int m = idx / Q, c = idx - m * Q;
            const int which = c / D, cc = c - which * D;
            float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
            if (m < nrows) {
                const float* up = which == 0 ? P.ai_gqs : (which == 1 ? P.ai_gk : P.ai_gv);
                if (up) v = *reinterpret_cast<const float4*>(up + (size_t)(r0 + m) * D + cc);
                if (which == 0) {
                    const float ga = s_ga[m * P.H + (cc >> 4)];
                    const float4 w4 = *reinterpret_cast<const float4*>(P.ai_w + cc);
                    v.x = fmaf(ga, w4.x, v.x * P.q_scale); v.y = fmaf(ga, w4.y, v.y * P.q_scale);
                    v.z = fmaf(ga, w4.z, v.z * P.q_scale); v.w = fmaf(ga, w4.w, v.w * P.q_scale);
                }
                *reinterpret_cast<float4*>(P.gqkv_out + (size_t)(r0 + m) * Q + c) = v;
            }
            *reinterpret_cast<float4*>(s_q + m * (Q + BR_PAD) + c) = v;
        }
        for (int c = threadIdx.x; c < D; c += 64 * BR_WAVES) {
            float sum = 0.0f;
#pragma unroll
            for (int m = 0; m < BR_ROWS; m++) sum = fmaf(s_ga[m * P.H + (c >> 4)], s_qf[m * ldd + c], sum);
            P.gw_partial[(size_t)blockIdx.x * D + c] = sum;
        }
        __syncthreads();
        bridge_bwd_products(s_q, Q, P.Wq, D, part);
        __syncthreads();
        bridge_bwd_finish(part, D, P.g_x2, nullptr, nullptr, r0, nrows, s_g2, P.g2);
    } else if (P.gqkv) {
        for (int idx = threadIdx.x * 4; idx < BR_ROWS * Q; idx += 64 * BR_WAVES * 4) {
            const int m = idx / Q, c = idx - m * Q;
            float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
            if (m < nrows) v = *reinterpret_cast<const float4*>(P.gqkv + (size_t)(r0 + m) * Q + c);
            *reinterpret_cast<float4*>(s_q + m * (Q + BR_PAD) + c) = v;
        }
        __syncthreads();
        bridge_bwd_products(s_q, Q, P.Wq, D, part);
        __syncthreads();
        bridge_bwd_finish(part, D, P.g_x2, nullptr, nullptr, r0, nrows, s_g2, P.g2);
    } else {
        for (int idx = threadIdx.x * 4; idx < BR_ROWS * D; idx += 64 * BR_WAVES * 4) {
            const int m = idx / D, c = idx - m * D;
            float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
            if (m < nrows && P.g_x2) v = *reinterpret_cast<const float4*>(P.g_x2 + (size_t)(r0 + m) * D + c);
            *reinterpret_cast<float4*>(s_g2 + m * (D + BR_PAD) + c) = v;
        }
    }
    __syncthreads();
    bridge_bwd_products(s_g2, D, P.W2, F, part);
    __syncthreads();
    bridge_bwd_finish(part, F, nullptr, nullptr, P.h, r0, nrows, s_gh, P.gh);
    __syncthreads();
    bridge_bwd_products(s_gh, F, P.W1, D, part);
    __syncthreads();
    bridge_bwd_finish(part, D, nullptr, s_g2, nullptr, r0, nrows, s_g1, P.g1);
    __syncthreads();
    bridge_bwd_products(s_g1, D, P.Wo, D, part);
    __syncthreads();
    bridge_bwd_finish(part, D, nullptr, nullptr, nullptr, r0, nrows, nullptr, P.g_attn);
}

}  // namespace cfh
