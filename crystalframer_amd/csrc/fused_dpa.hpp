// Softmax-over-neighbours attention with per-pair logit bias and per-pair value bias, and the
// per-crystal mean.  The reference's counterparts are models/kernels/fused_dpa_fwd.cu,
// fused_dpa_bwd.cu, fused_dpa_bwd_q.cu, irregular_transpose.cu (driven by
// models/cuda_funcs/fused_dpa.py:17-170) and models/kernels/irregular_mean_fwd.cu
// (models/cuda_funcs/irregular_mean.py:19-70).
//
//   l_e = q_i . k_j + a_e,   p_e = softmax over the pairs e = (i, .) of atom i,
//   o_i = sum_e p_e (v_j + b_e)
//
// One wavefront per (atom, head).  A lane is (slot, channel): 4 pairs are in flight at once, each
// on 16 lanes that hold one channel of the 16-wide head each.  The forward keeps a running
// (max, sum, accumulator) per slot and merges the four slots at the end, so a row of any length
// needs no scratch memory.  The backward is split in a row kernel (gq, ga, gb: everything indexed
// like the forward) and a column kernel (gk, gv: sums over the pairs (., j) that point AT an atom),
// which finds the pair (i, j) from the row of i.  Pairs are the complete n x n block of each
// crystal, rows and columns in atom order -- the layout the reference's transposition kernel
// assumes as well -- so pair (i, j) sits at e_start[i] + (j - first atom of the crystal).
// Every sum is taken in a fixed order: results are bit-reproducible run to run.
#pragma once
#include "device_common.hpp"

namespace cfh {

struct DpaArgs {
    const float* q;          // (N,H,16), already divided by sqrt(16)
    const float* k;          // (N,H,16)
    const float* v;          // (N,H,16)
    const float* aij;        // (E,H) or null
    const float* bij;        // (E,H,16) or null
    const int64_t* edges;    // (2,E)
    const int64_t* e_start;  // (N+1)
    float* prob;             // (E,H)  forward: out, backward: in
    float* out;              // (N,H,16) forward: out, backward: in
    const float* go;         // (N,H,16)
    float* gq;
    float* gk;
    float* gv;
    float* gaij;             // (E,H): always written by the row kernel, read by the column kernel
    float* gbij;             // (E,H,16) or null
    int32_t N, H, E;
};

constexpr int DPA_WAVES = 4;     // wavefronts (items) per workgroup

// sum over the 16 lanes of a slot
__device__ __forceinline__ float slot_sum(float x) {
    x += __shfl_xor(x, 1, WAVE);
    x += __shfl_xor(x, 2, WAVE);
    x += __shfl_xor(x, 4, WAVE);
    x += __shfl_xor(x, 8, WAVE);
    return x;
}

__global__ __launch_bounds__(WAVE * DPA_WAVES) void dpa_fwd_kernel(const DpaArgs P) {
    const int lane = threadIdx.x & (WAVE - 1);
    const int item = blockIdx.x * DPA_WAVES + (threadIdx.x >> 6);
    if (item >= P.N * P.H) return;
    const int H = P.H;
    const int i = item / H, h = item - i * H;
    const int slot = lane >> 4, c = lane & 15;
    const int e0 = (int)P.e_start[i], e1 = (int)P.e_start[i + 1];
    const float qc = P.q[((size_t)i * H + h) * DH + c];

    float m = -3.0e38f, s = 0.0f, acc = 0.0f;
    for (int eb = e0; eb < e1; eb += 4) {
        const int e = eb + slot;
        const bool valid = e < e1;
        float part = 0.0f, val = 0.0f, bias = 0.0f;
        if (valid) {
            const size_t j = (size_t)P.edges[(size_t)P.E + e];
            part = qc * P.k[(j * H + h) * DH + c];
            val = P.v[(j * H + h) * DH + c];
            if (P.bij) val += P.bij[((size_t)e * H + h) * DH + c];
            if (P.aij) bias = P.aij[(size_t)e * H + h];
        }
        const float l = slot_sum(part) + bias;
        if (valid) {
            if (c == 0) P.prob[(size_t)e * H + h] = l;       // the logit for now
            const float mn = fmaxf(m, l);
            const float sc = __expf(m - mn), w = __expf(l - mn);
            s = s * sc + w;
            acc = acc * sc + w * val;
            m = mn;
        }
    }
    // merge the four slots
    float M = fmaxf(m, __shfl_xor(m, 16, WAVE));
    M = fmaxf(M, __shfl_xor(M, 32, WAVE));
    const float sc = (s > 0.0f) ? __expf(m - M) : 0.0f;
    s *= sc; acc *= sc;
    s += __shfl_xor(s, 16, WAVE); s += __shfl_xor(s, 32, WAVE);
    acc += __shfl_xor(acc, 16, WAVE); acc += __shfl_xor(acc, 32, WAVE);
    const float inv = (s > 0.0f) ? 1.0f / s : 0.0f;
    if (slot == 0) P.out[((size_t)i * H + h) * DH + c] = acc * inv;
    // logits -> probabilities (each was written by the lane that now reads it)
    if (c == 0)
        for (int e = e0 + slot; e < e1; e += 4) {
            const size_t o = (size_t)e * H + h;
            P.prob[o] = __expf(P.prob[o] - M) * inv;
        }
}

// gq_i = sum_e gl_e k_j, ga_e = gl_e = p_e (go_i.(v_j + b_e) - go_i.o_i), gb_e = p_e go_i
__global__ __launch_bounds__(WAVE * DPA_WAVES) void dpa_bwd_row_kernel(const DpaArgs P) {
    const int lane = threadIdx.x & (WAVE - 1);
    const int item = blockIdx.x * DPA_WAVES + (threadIdx.x >> 6);
    if (item >= P.N * P.H) return;
    const int H = P.H;
    const int i = item / H, h = item - i * H;
    const int slot = lane >> 4, c = lane & 15;
    const int e0 = (int)P.e_start[i], e1 = (int)P.e_start[i + 1];
    const size_t ih = ((size_t)i * H + h) * DH + c;
    const float goc = P.go[ih];
    const float D = slot_sum(goc * P.out[ih]);
    float gq = 0.0f;
    for (int eb = e0; eb < e1; eb += 4) {
        const int e = eb + slot;
        const bool valid = e < e1;
        float part = 0.0f, kc = 0.0f, p = 0.0f;
        if (valid) {
            const size_t j = (size_t)P.edges[(size_t)P.E + e];
            kc = P.k[(j * H + h) * DH + c];
            float val = P.v[(j * H + h) * DH + c];
            if (P.bij) val += P.bij[((size_t)e * H + h) * DH + c];
            p = P.prob[(size_t)e * H + h];
            part = goc * val;
        }
        const float gl = p * (slot_sum(part) - D);
        if (valid) {
            if (c == 0) P.gaij[(size_t)e * H + h] = gl;
            if (P.gbij) P.gbij[((size_t)e * H + h) * DH + c] = p * goc;
            gq = fmaf(gl, kc, gq);
        }
    }
    gq += __shfl_xor(gq, 16, WAVE);
    gq += __shfl_xor(gq, 32, WAVE);
    if (slot == 0) P.gq[ih] = gq;
}

// gk_j = sum_i gl_(i,j) q_i, gv_j = sum_i p_(i,j) go_i over the atoms i of the crystal of j
__global__ __launch_bounds__(WAVE * DPA_WAVES) void dpa_bwd_col_kernel(const DpaArgs P) {
    const int lane = threadIdx.x & (WAVE - 1);
    const int item = blockIdx.x * DPA_WAVES + (threadIdx.x >> 6);
    if (item >= P.N * P.H) return;
    const int H = P.H;
    const int j = item / H, h = item - j * H;
    const int slot = lane >> 4, c = lane & 15;
    const int e0 = (int)P.e_start[j], n = (int)P.e_start[j + 1] - e0;
    float gk = 0.0f, gv = 0.0f;
    if (n > 0) {
        const int first = (int)P.edges[(size_t)P.E + e0];      // first atom of the crystal
        const int col = j - first;
        for (int ib = 0; ib < n; ib += 4) {
            const int r = ib + slot;
            if (r < n) {
                const int i = first + r;
                const size_t e = (size_t)P.e_start[i] + col;
                const size_t ih = ((size_t)i * H + h) * DH + c;
                gk = fmaf(P.gaij[e * H + h], P.q[ih], gk);
                gv = fmaf(P.prob[e * H + h], P.go[ih], gv);
            }
        }
    }
    gk += __shfl_xor(gk, 16, WAVE); gk += __shfl_xor(gk, 32, WAVE);
    gv += __shfl_xor(gv, 16, WAVE); gv += __shfl_xor(gv, 32, WAVE);
    if (slot == 0) {
        const size_t jh = ((size_t)j * H + h) * DH + c;
        P.gk[jh] = gk;
        P.gv[jh] = gv;
    }
}

__global__ void set_flag_kernel(int* flag, int value) { *flag = value; }

// 1 where the pairs are not the complete n x n block of each crystal in atom order, else untouched
__global__ void dpa_check_layout_kernel(const int64_t* edges, const int64_t* e_start, int N, int E, int* bad) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= N) return;
    const int e0 = (int)e_start[i], e1 = (int)e_start[i + 1];
    if (e1 <= e0) return;
    const int64_t first = edges[(size_t)E + e0];
    bool ok = first >= 0 && first + (e1 - e0) <= N && i >= first && i < first + (e1 - e0);
    for (int e = e0; ok && e < e1; e++)
        ok = edges[e] == i && edges[(size_t)E + e] == first + (e - e0);
    if (ok) {
        // every atom of the crystal must see the same block
        const int64_t f0 = e_start[first];
        ok = e_start[first + 1] - f0 == e1 - e0 && edges[(size_t)E + f0] == first;
    }
    if (!ok) *bad = 1;
}

// out[b, c] = mean over the atoms of crystal b of x[i, c]
__global__ void crystal_mean_fwd_kernel(const float* x, const int64_t* atom_start, int B, int C, float* out) {
    const int b = blockIdx.x;
    const int64_t s = atom_start[b], t = atom_start[b + 1];
    const float inv = t > s ? 1.0f / (float)(t - s) : 0.0f;
    for (int c = threadIdx.x; c < C; c += blockDim.x) {
        float acc = 0.0f;
        for (int64_t i = s; i < t; i++) acc += x[(size_t)i * C + c];
        out[(size_t)b * C + c] = acc * inv;
    }
}

// gx[i, c] = gout[batch[i], c] / size of the crystal
__global__ void crystal_mean_bwd_kernel(const float* gout, const int64_t* batch, const int64_t* atom_start,
                                        int N, int C, float* gx) {
    const size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= (size_t)N * C) return;
    const int i = (int)(idx / C), c = (int)(idx - (size_t)i * C);
    const int64_t b = batch[i];
    const float inv = 1.0f / (float)(atom_start[b + 1] - atom_start[b]);
    gx[idx] = gout[(size_t)b * C + c] * inv;
}

}  // namespace cfh
