// Forward of the framed value position encoding: z, psi (and optionally d2min) for every
// (pair, head).  One launch covers what the reference does in two kernels plus a tensor sum
// (models/kernels/real_enc_frame_proj_fwd_length.cu, ..._fwd_angle.cu,
//  models/cuda_funcs/real_space_framed_proj.py:63-105).
//
// Per pair e=(i,j) and head h, with lanes running over translations n:
//   pass A  d2min = min_n |r_ij + n.L|^2                                  (6 VALU per translation)
//   pass B  keep the translations with a(d^2-d2min) >= -prune (ballot/prefix compaction into LDS)
//   pass C  for kept n: w = 2^(a'(d^2-d2min)); S += w; scatter w*g_k(d) into the 9-bin distance
//           window and w*g_m(cos(n, f_axis)) into the three 33-bin angle windows (LDS float adds,
//           Gaussians by recurrence)
//   epilogue lane (enc,c): psi_enc[c] = W_enc[h,c,:] . hist_enc / S, W rows held in registers;
//           z = log S + a d2min.
#pragma once
#include "device_common.hpp"

namespace cfh {

template <int WL, int WA, bool COS_ABS, bool HAS_LEN, bool HAS_ANG>
__global__ __launch_bounds__(WAVE) void framed_pe_fwd_kernel(const KernelArgs P) {
    __shared__ float4 tab[TCAP];
    __shared__ uint16_t list[TCAP];
    __shared__ __attribute__((aligned(16))) float hist[4 * HS];

    const int lane = threadIdx.x;
    const int H = P.H;
    const int h = blockIdx.x % H;
    const int enc = lane >> 4;        // 0 = distance, 1..3 = frame axes
    const int c = lane & 15;          // output channel

    // this lane's row of the projection weights, W_enc[h, c, 0:64]
    float Wrow[NBINS];
    {
        const bool used = (enc == 0) ? HAS_LEN : HAS_ANG;
        const float* src = used ? P.W[enc] + ((size_t)h * DH + c) * NBINS : nullptr;
#pragma unroll
        for (int k4 = 0; k4 < NBINS / 4; k4++) {
            float4 v = used ? reinterpret_cast<const float4*>(src)[k4] : make_float4(0.f, 0.f, 0.f, 0.f);
            Wrow[4 * k4 + 0] = v.x; Wrow[4 * k4 + 1] = v.y; Wrow[4 * k4 + 2] = v.z; Wrow[4 * k4 + 3] = v.w;
        }
    }
    const float enc_coef = (enc == 0) ? P.dist_coef : P.angle_coef;
    const BasisConsts bc = P.bc;
    const float prune = (P.prune_log2 > 0.0f) ? -P.prune_log2 : -3.0e38f;

    for (;;) {
        const int it = next_item(P.counters + h, lane);
        if (it >= P.N) break;
        const int i = P.order ? uniform_i(P.order[it]) : it;
        const int b = uniform_i((int)P.batch[i]);
        const float a = uniform_f(P.a_ih[(size_t)i * H + h]);
        const float a2 = a * LOG2E;
        Lattice L;
#pragma unroll
        for (int d = 0; d < 9; d++) L.t[d] = uniform_f(P.tvecs[(size_t)b * 9 + d]);
        float rvl1 = 0.f, rvl2 = 0.f, rvl3 = 0.f;
        if (P.rvlen) {
            rvl1 = uniform_f(P.rvlen[(size_t)b * 3 + 0]);
            rvl2 = uniform_f(P.rvlen[(size_t)b * 3 + 1]);
            rvl3 = uniform_f(P.rvlen[(size_t)b * 3 + 2]);
        }
        const Box bx = translation_box(a, rvl1, rvl2, rvl3, P.cutoff_radius, P.lattice_range,
                                       P.minimum_range);
        float f[3][3];
        if (HAS_ANG) {
#pragma unroll
            for (int ax = 0; ax < 3; ax++)
#pragma unroll
                for (int d = 0; d < 3; d++)
                    f[ax][d] = uniform_f(P.frames[(((size_t)ax * P.N + i) * H + h) * 3 + d]);
        }
        const int nchunks = (bx.T + TCAP - 1) / TCAP;
        if (nchunks == 1) {
            __syncthreads();
            build_shift_table(tab, 0, bx.T, bx, L, lane);
            __syncthreads();
        }
        const int e0 = uniform_i((int)P.e_start[i]);
        const int e1 = uniform_i((int)P.e_start[i + 1]);

        for (int e = e0; e < e1; e++) {
            const float rx = uniform_f(P.rpos[(size_t)e * 3 + 0]);
            const float ry = uniform_f(P.rpos[(size_t)e * 3 + 1]);
            const float rz = uniform_f(P.rpos[(size_t)e * 3 + 2]);

            // ---- pass A: nearest image
            float d2min = 3.0e38f;
            for (int ch = 0; ch < nchunks; ch++) {
                const int t0 = ch * TCAP;
                const int cnt = min(TCAP, bx.T - t0);
                if (nchunks > 1) {
                    __syncthreads();
                    build_shift_table(tab, t0, cnt, bx, L, lane);
                    __syncthreads();
                }
                for (int u = lane; u < cnt; u += WAVE) {
                    const float4 v = tab[u];
                    const float dx = rx + v.x, dy = ry + v.y, dz = rz + v.z;
                    d2min = fminf(d2min, fmaf(dx, dx, fmaf(dy, dy, dz * dz)));
                }
            }
            d2min = wave_min(d2min);

            // ---- clear the histograms
            __syncthreads();
            for (int u = lane; u < 4 * HS; u += WAVE) hist[u] = 0.0f;
            __syncthreads();

            float S = 0.0f;
            for (int ch = 0; ch < nchunks; ch++) {
                const int t0 = ch * TCAP;
                const int cnt = min(TCAP, bx.T - t0);
                if (nchunks > 1) {
                    __syncthreads();
                    build_shift_table(tab, t0, cnt, bx, L, lane);
                    __syncthreads();
                }
                // ---- pass B: compaction of the translations that matter
                int nkeep = 0;
                for (int u0 = 0; u0 < cnt; u0 += WAVE) {
                    const int u = u0 + lane;
                    bool keep = false;
                    if (u < cnt) {
                        const float4 v = tab[u];
                        const float dx = rx + v.x, dy = ry + v.y, dz = rz + v.z;
                        const float d2 = fmaf(dx, dx, fmaf(dy, dy, dz * dz));
                        keep = a2 * (d2 - d2min) >= prune;
                    }
                    const uint64_t m = __ballot(keep);
                    if (keep) list[nkeep + lane_prefix(m)] = (uint16_t)u;
                    nkeep += __popcll(m);
                }
                __syncthreads();
                // ---- pass C: weights and window scatters
                for (int v0 = 0; v0 < nkeep; v0 += WAVE) {
                    if (v0 + lane < nkeep) {
                        const float4 v = tab[list[v0 + lane]];
                        const float dx = rx + v.x, dy = ry + v.y, dz = rz + v.z;
                        const float d2 = fmaf(dx, dx, fmaf(dy, dy, dz * dz));
                        const float w = hw_exp2(a2 * (d2 - d2min));
                        S += w;
                        if (HAS_LEN) {
                            const float d = hw_sqrt(d2);
                            const float u = d * bc.inv_interval;
                            int start = (int)(u - bc.start_off);          // truncation toward zero
                            start = max(0, min(start, NBINS - WL));
                            // bin k has centre (k+1)*interval: scaled offset ((k+1) - u)*len_step
                            const float beta_c = ((float)(start + WL / 2 + 1) - u) * bc.len_step;
                            const WindowSeed s = window_seed(beta_c, bc.len_step, w);
                            window_scatter<WL>(hist + start, s, bc.len_cc);
                        }
                        if (HAS_ANG) {
                            if (d2 > 1e-5f) {       // the self image contributes to S only
                                const float rinv = hw_rsq(d2);
#pragma unroll
                                for (int ax = 0; ax < 3; ax++) {
                                    float cs = (dx * f[ax][0] + dy * f[ax][1] + dz * f[ax][2]) * rinv;
                                    if (COS_ABS) cs = fabsf(cs);
                                    int end = (int)fminf((cs + bc.ang_end_off) * bc.ang_inv_interval + 1.0f,
                                                         (float)NBINS);
                                    end = max(end, WA);
                                    const int start = end - WA;
                                    const float mu_c = bc.ang_mu0 + (float)(start + WA / 2) * bc.ang_interval;
                                    const float beta_c = (mu_c - cs) * bc.ang_sigma_inv;
                                    const WindowSeed s = window_seed(beta_c, bc.ang_step, w);
                                    window_scatter<WA>(hist + (ax + 1) * HS + start, s, bc.ang_cc);
                                }
                            }
                        }
                    }
                }
                __syncthreads();
            }
            S = wave_sum(S);

            // ---- epilogue: projection by this lane's weight row
            const float inv_S = 1.0f / S;
            float acc = 0.0f;
            if (HAS_LEN || HAS_ANG) {
                const float4* hrow = reinterpret_cast<const float4*>(hist + enc * HS);
#pragma unroll
                for (int k4 = 0; k4 < NBINS / 4; k4++) {
                    const float4 hv = hrow[k4];
                    acc = fmaf(Wrow[4 * k4 + 0], hv.x, acc);
                    acc = fmaf(Wrow[4 * k4 + 1], hv.y, acc);
                    acc = fmaf(Wrow[4 * k4 + 2], hv.z, acc);
                    acc = fmaf(Wrow[4 * k4 + 3], hv.w, acc);
                }
                acc *= inv_S * enc_coef;
                acc += __shfl_xor(acc, 16, WAVE);
                acc += __shfl_xor(acc, 32, WAVE);
                if (lane < DH && P.out_psi) P.out_psi[((size_t)e * H + h) * DH + lane] = acc;
            }
            if (lane == 0) {
                P.out_z[(size_t)e * H + h] = logf(S) + d2min * a;
                if (P.out_d2min) P.out_d2min[(size_t)e * H + h] = d2min;
            }
        }
    }
}

}  // namespace cfh
