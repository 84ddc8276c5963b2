// Softmax-over-neighbours attention with per-pair logit bias and per-pair value bias, and the
// per-crystal mean.  The reference's counterparts are models/kernels/fused_dpa_fwd.cu,
// fused_dpa_bwd.cu, fused_dpa_bwd_q.cu, irregular_transpose.cu (driven by
// models/cuda_funcs/fused_dpa.py:17-170) and models/kernels/irregular_mean_fwd.cu
// (models/cuda_funcs/irregular_mean.py:19-70).
//
//   l_e = q_i . k_j + a_e,   p_e = softmax over the pairs e = (i, .) of atom i,
//   o_i = sum_e p_e (v_j + b_e)
//
// One wavefront per (atom, head).  A lane is (slot, quarter): 16 pairs are in flight at once, each
// on 4 lanes that hold 4 of the 16 channels of the head each (one 16-byte load per lane and operand;
// most rows fit one step, so a row costs three dependent memory round trips: its bounds, the
// neighbour indices, the operands).  Rows of up to 16 pairs are finished in registers; longer rows
// keep a running (max, sum, accumulator) per slot, merge the slots at the end and rescale the
// logits they parked in the probability array.  The backward is split in a row kernel (gq, ga, gb:
// everything indexed like the forward) and a column kernel (gk, gv: sums over the pairs (., j) that
// point AT an atom), which finds the pair (i, j) from the row of i.  Pairs are the complete n x n
// block of each crystal, rows and columns in atom order -- the layout the reference's transposition
// kernel assumes as well -- so pair (i, j) sits at e_start[i] + (j - first atom of the crystal).
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
    const uint32_t* items;   // optional (column kernel): the item records (N, H, REC_WORDS) of the launch before, in work
                             // order; they hold an atom's first pair, pair count and first neighbour in one place
};

constexpr int DPA_WAVES = 4;     // wavefronts (items) per workgroup
constexpr int DPA_SLOTS = 16;    // pairs in flight per wavefront

// sum over the 4 lanes of a slot (quad_perm [1,0,3,2], [2,3,0,1])
__device__ __forceinline__ float quad_sum(float x) {
    x += dpp_move<0xB1>(x);
    x += dpp_move<0x4E>(x);
    return x;
}
// sum over the 16 slots, for every quarter: lanes q, q+4, ..., q+60 (row_ror 4, 8, then the four rows)
__device__ __forceinline__ float slots_sum(float x) {
    x += dpp_move<0x124>(x);
    x += dpp_move<0x128>(x);
    return rows_sum(x);
}
__device__ __forceinline__ float4 slots_sum(float4 v) {
    return make_float4(slots_sum(v.x), slots_sum(v.y), slots_sum(v.z), slots_sum(v.w));
}
__device__ __forceinline__ float wave_max(float v) { return -wave_min(-v); }
__device__ __forceinline__ float dot4(const float4& a, const float4& b) {
    return fmaf(a.x, b.x, fmaf(a.y, b.y, fmaf(a.z, b.z, a.w * b.w)));
}
__device__ __forceinline__ float4 ld4(const float* base, size_t row, int quarter) {
    return reinterpret_cast<const float4*>(base + row * DH)[quarter];
}

__global__ __launch_bounds__(WAVE * DPA_WAVES) void dpa_fwd_kernel(const DpaArgs P) {
    const int lane = threadIdx.x & (WAVE - 1);
    const int item = blockIdx.x * DPA_WAVES + (threadIdx.x >> 6);
    if (item >= P.N * P.H) return;
    const int H = P.H;
    const int i = item / H, h = item - i * H;
    const int slot = lane >> 2, qd = lane & 3;
    const int e0 = (int)P.e_start[i], e1 = (int)P.e_start[i + 1];
    const float4 q4 = ld4(P.q, (size_t)i * H + h, qd);
    float4* const out4 = reinterpret_cast<float4*>(P.out + ((size_t)i * H + h) * DH) + qd;

    if (e1 - e0 <= DPA_SLOTS) {
        // the whole row in one step
        const int e = e0 + slot;
        const bool valid = e < e1;
        float part = 0.0f, bias = 0.0f;
        float4 val = make_float4(0.f, 0.f, 0.f, 0.f);
        if (valid) {
            const size_t j = (size_t)P.edges[(size_t)P.E + e];
            part = dot4(q4, ld4(P.k, j * H + h, qd));
            val = ld4(P.v, j * H + h, qd);
            if (P.bij) {
                const float4 b = ld4(P.bij, (size_t)e * H + h, qd);
                val.x += b.x; val.y += b.y; val.z += b.z; val.w += b.w;
            }
            if (P.aij) bias = P.aij[(size_t)e * H + h];
        }
        const float l = valid ? quad_sum(part) + bias : -3.0e38f;
        const float M = wave_max(l);
        const float w = valid ? __expf(l - M) : 0.0f;
        const float S = wave_sum(w) * 0.25f;              // every slot counted by its 4 lanes
        const float inv = (S > 0.0f) ? 1.0f / S : 0.0f;
        const float4 acc = slots_sum(make_float4(w * val.x, w * val.y, w * val.z, w * val.w));
        if (slot == 0) *out4 = make_float4(acc.x * inv, acc.y * inv, acc.z * inv, acc.w * inv);
        if (valid && qd == 0) P.prob[(size_t)e * H + h] = w * inv;
        return;
    }

    float m = -3.0e38f, s = 0.0f;
    float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
    for (int eb = e0; eb < e1; eb += DPA_SLOTS) {
        const int e = eb + slot;
        const bool valid = e < e1;
        float part = 0.0f, bias = 0.0f;
        float4 val = make_float4(0.f, 0.f, 0.f, 0.f);
        if (valid) {
            const size_t j = (size_t)P.edges[(size_t)P.E + e];
            part = dot4(q4, ld4(P.k, j * H + h, qd));
            val = ld4(P.v, j * H + h, qd);
            if (P.bij) {
                const float4 b = ld4(P.bij, (size_t)e * H + h, qd);
                val.x += b.x; val.y += b.y; val.z += b.z; val.w += b.w;
            }
            if (P.aij) bias = P.aij[(size_t)e * H + h];
        }
        const float l = quad_sum(part) + bias;
        if (valid) {
            if (qd == 0) P.prob[(size_t)e * H + h] = l;       // the logit for now
            const float mn = fmaxf(m, l);
            const float sc = __expf(m - mn), w = __expf(l - mn);
            s = s * sc + w;
            acc.x = acc.x * sc + w * val.x; acc.y = acc.y * sc + w * val.y;
            acc.z = acc.z * sc + w * val.z; acc.w = acc.w * sc + w * val.w;
            m = mn;
        }
    }
    // merge the slots
    const float M = wave_max(m);
    const float sc = (s > 0.0f) ? __expf(m - M) : 0.0f;
    const float S = wave_sum(s * sc) * 0.25f;
    const float inv = (S > 0.0f) ? 1.0f / S : 0.0f;
    acc = slots_sum(make_float4(acc.x * sc, acc.y * sc, acc.z * sc, acc.w * sc));
    if (slot == 0) *out4 = make_float4(acc.x * inv, acc.y * inv, acc.z * inv, acc.w * inv);
    // logits -> probabilities (each was written by the lane that now reads it)
    if (qd == 0)
        for (int e = e0 + slot; e < e1; e += DPA_SLOTS) {
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
    const int slot = lane >> 2, qd = lane & 3;
    const int e0 = (int)P.e_start[i], e1 = (int)P.e_start[i + 1];
    const size_t ih = (size_t)i * H + h;
    const float4 go4 = ld4(P.go, ih, qd);
    const float D = quad_sum(dot4(go4, ld4(P.out, ih, qd)));
    float4 gq = make_float4(0.f, 0.f, 0.f, 0.f);
    for (int eb = e0; eb < e1; eb += DPA_SLOTS) {
        const int e = eb + slot;
        const bool valid = e < e1;
        float part = 0.0f, p = 0.0f;
        float4 k4 = make_float4(0.f, 0.f, 0.f, 0.f);
        if (valid) {
            const size_t j = (size_t)P.edges[(size_t)P.E + e];
            k4 = ld4(P.k, j * H + h, qd);
            float4 val = ld4(P.v, j * H + h, qd);
            if (P.bij) {
                const float4 b = ld4(P.bij, (size_t)e * H + h, qd);
                val.x += b.x; val.y += b.y; val.z += b.z; val.w += b.w;
            }
            p = P.prob[(size_t)e * H + h];
            part = dot4(go4, val);
        }
        const float gl = p * (quad_sum(part) - D);
        if (valid) {
            if (qd == 0) P.gaij[(size_t)e * H + h] = gl;
            if (P.gbij)
                reinterpret_cast<float4*>(P.gbij + ((size_t)e * H + h) * DH)[qd] =
                    make_float4(p * go4.x, p * go4.y, p * go4.z, p * go4.w);
            gq.x = fmaf(gl, k4.x, gq.x); gq.y = fmaf(gl, k4.y, gq.y);
            gq.z = fmaf(gl, k4.z, gq.z); gq.w = fmaf(gl, k4.w, gq.w);
        }
    }
    gq = slots_sum(gq);
    if (slot == 0) reinterpret_cast<float4*>(P.gq + ih * DH)[qd] = gq;
}

// gk_j = sum_i gl_(i,j) q_i, gv_j = sum_i p_(i,j) go_i over the atoms i of the crystal of j; every
// row of the crystal's block has n pairs, so pair (i, j) is at (first pair of the crystal) + r n + col
__global__ __launch_bounds__(WAVE * DPA_WAVES) void dpa_bwd_col_kernel(const DpaArgs P) {
    const int lane = threadIdx.x & (WAVE - 1);
    const int item = blockIdx.x * DPA_WAVES + (threadIdx.x >> 6);
    if (item >= P.N * P.H) return;
    const int H = P.H;
    int j = item / H;
    const int h = item - j * H;
    const int slot = lane >> 2, qd = lane & 3;
    int e0, n, first = 0;
    if (P.items) {
        // (the atoms in work order instead of atom order: one read where the arrays need two that wait for each other)
        const uint4 r4 = *reinterpret_cast<const uint4*>(P.items + (size_t)item * REC_WORDS);
        j = (int)r4.x; e0 = (int)r4.y; n = (int)r4.z;
        first = (int)P.items[(size_t)item * REC_WORDS + 30];
    } else {
        e0 = (int)P.e_start[j];
        n = (int)P.e_start[j + 1] - e0;
        if (n > 0) first = (int)P.edges[(size_t)P.E + e0];      // first atom of the crystal
    }
    float4 gk = make_float4(0.f, 0.f, 0.f, 0.f), gv = gk;
    if (n > 0) {
        const int col = j - first;
        const size_t eblock = (size_t)e0 - (size_t)col * n;    // first pair of the crystal
        for (int ib = 0; ib < n; ib += DPA_SLOTS) {
            const int r = ib + slot;
            if (r < n) {
                const size_t e = eblock + (size_t)r * n + col;
                const size_t ih = (size_t)(first + r) * H + h;
                const float gl = P.gaij[e * H + h], p = P.prob[e * H + h];
                const float4 q4 = ld4(P.q, ih, qd), go4 = ld4(P.go, ih, qd);
                gk.x = fmaf(gl, q4.x, gk.x); gk.y = fmaf(gl, q4.y, gk.y);
                gk.z = fmaf(gl, q4.z, gk.z); gk.w = fmaf(gl, q4.w, gk.w);
                gv.x = fmaf(p, go4.x, gv.x); gv.y = fmaf(p, go4.y, gv.y);
                gv.z = fmaf(p, go4.z, gv.z); gv.w = fmaf(p, go4.w, gv.w);
            }
        }
    }
    gk = slots_sum(gk);
    gv = slots_sum(gv);
    if (slot == 0) {
        const size_t jh = (size_t)j * H + h;
        reinterpret_cast<float4*>(P.gk + jh * DH)[qd] = gk;
        reinterpret_cast<float4*>(P.gv + jh * DH)[qd] = gv;
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

// The same for rows of C = 4 Q floats, Q <= 256, 16-byte aligned: a block of 256 threads per crystal, thread =
// (slice of the atoms, four channels as one 16-byte load), the 256 / Q slices added up in LDS in a fixed order.
__global__ __launch_bounds__(256) void crystal_mean_fwd_vec_kernel(const float* x, const int64_t* atom_start, int B,
                                                                   int C, float* out) {
    __shared__ float4 part[256];
    const int b = blockIdx.x;
    const int Q = C >> 2, S = 256 / Q;
    const int q = threadIdx.x % Q, sl = threadIdx.x / Q;
    const int64_t s = atom_start[b], t = atom_start[b + 1];
    const float4* const x4 = reinterpret_cast<const float4*>(x);
    float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
    if (sl < S)
        for (int64_t i = s + sl; i < t; i += S) {
            const float4 v = x4[(size_t)i * Q + q];
            acc.x += v.x; acc.y += v.y; acc.z += v.z; acc.w += v.w;
        }
    part[threadIdx.x] = acc;
    __syncthreads();
    if (threadIdx.x < Q) {
        for (int k = 1; k < S; k++) {
            const float4 v = part[k * Q + q];
            acc.x += v.x; acc.y += v.y; acc.z += v.z; acc.w += v.w;
        }
        const float inv = t > s ? 1.0f / (float)(t - s) : 0.0f;
        reinterpret_cast<float4*>(out)[(size_t)b * Q + q] = make_float4(acc.x * inv, acc.y * inv, acc.z * inv, acc.w * inv);
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
