// Forward of the framed value position encoding: z, psi (and optionally d2min) for every
// (pair, head).  One launch covers what the reference does in two kernels plus a tensor sum
// (models/kernels/real_enc_frame_proj_fwd_length.cu, ..._fwd_angle.cu,
//  models/cuda_funcs/real_space_framed_proj.py:63-105).
//
// Per pair e=(i,j) and head h, with lanes running over translations n:
//   pass A  d2min = min_n |r_ij + n.L|^2                                  (6 VALU per translation)
//   pass B  w_n = 2^(a'(d^2-d2min)); S = sum_n w_n; the translations with w_n >= 2^-prune are
//           compacted (ballot/prefix) into an LDS list
//   pass C  for kept n: p = w/S; scatter p*g_k(d) into the 9-bin distance window and
//           p*g_m(cos(n, f_axis)) into the three 33-bin angle windows (fixed-point LDS adds,
//           Gaussians by recurrence)
//   epilogue lane (enc,c): psi_enc[c] = W_enc[h,c,:] . hist_enc, W rows held in registers;
//           z = log S + a d2min.
#pragma once
#include "device_common.hpp"

namespace cfh {

template <int WL, int WA, bool COS_ABS, bool HAS_LEN, bool HAS_ANG>
__global__ __launch_bounds__(WAVE) void framed_pe_fwd_kernel(const KernelArgs P) {
    __shared__ float4 tab[TCAP];
    __shared__ uint16_t list[TCAP];
    __shared__ uint32_t hist[NREP * REP_STRIDE];
    __shared__ __attribute__((aligned(16))) float shat[4 * HS];

    const int lane = threadIdx.x;
    const int H = P.H;
    const int h = blockIdx.x % H;
    const int enc = lane >> 4;        // 0 = distance, 1..3 = frame axes
    const int c = lane & 15;          // output channel
    uint32_t* const myhist = hist + (lane & (NREP - 1)) * REP_STRIDE;

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

    for (int u = lane; u < NREP * REP_STRIDE; u += WAVE) hist[u] = 0u;
    __syncthreads();

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
        unsigned long long n_eval = 0;

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

            // ---- the normaliser S when the table does not fit at once (otherwise pass B gives it)
            float S = 0.0f;
            if (nchunks > 1) {
                for (int ch = 0; ch < nchunks; ch++) {
                    const int t0 = ch * TCAP;
                    const int cnt = min(TCAP, bx.T - t0);
                    __syncthreads();
                    build_shift_table(tab, t0, cnt, bx, L, lane);
                    __syncthreads();
                    for (int u = lane; u < cnt; u += WAVE) {
                        const float4 v = tab[u];
                        const float dx = rx + v.x, dy = ry + v.y, dz = rz + v.z;
                        S += hw_exp2(a2 * (fmaf(dx, dx, fmaf(dy, dy, dz * dz)) - d2min));
                    }
                }
                S = wave_sum(S);
            }

            for (int ch = 0; ch < nchunks; ch++) {
                const int t0 = ch * TCAP;
                const int cnt = min(TCAP, bx.T - t0);
                if (nchunks > 1) {
                    __syncthreads();
                    build_shift_table(tab, t0, cnt, bx, L, lane);
                    __syncthreads();
                }
                // ---- pass B: weights, normaliser, compaction of the translations that matter
                int nkeep = 0;
                float Sb = 0.0f;
                for (int u0 = 0; u0 < cnt; u0 += WAVE) {
                    const int u = u0 + lane;
                    bool keep = false;
                    if (u < cnt) {
                        const float4 v = tab[u];
                        const float dx = rx + v.x, dy = ry + v.y, dz = rz + v.z;
                        const float ex = a2 * (fmaf(dx, dx, fmaf(dy, dy, dz * dz)) - d2min);
                        Sb += hw_exp2(ex);
                        keep = ex >= prune;
                    }
                    const uint64_t m = __ballot(keep);
                    if (keep) list[nkeep + lane_prefix(m)] = (uint16_t)u;
                    nkeep += __popcll(m);
                }
                if (nchunks == 1) S = wave_sum(Sb);
                n_eval += (unsigned long long)nkeep;
                const float wfix = FIX_ONE / S;
                __syncthreads();
                // ---- pass C: window scatters of the normalised weights
                if (HAS_LEN) {
                    for (int v0 = 0; v0 < nkeep; v0 += WAVE) {
                        if (v0 + lane < nkeep) {
                            const float4 v = tab[list[v0 + lane]];
                            const float dx = rx + v.x, dy = ry + v.y, dz = rz + v.z;
                            const float d2 = fmaf(dx, dx, fmaf(dy, dy, dz * dz));
                            const float w = hw_exp2(a2 * (d2 - d2min)) * wfix;
                            {
                                const float d = hw_sqrt(d2);
                                const float u = d * bc.inv_interval;
                                int start = (int)(u - bc.start_off);          // truncation toward zero
                                start = max(0, min(start, NBINS - WL));
                                // bin k has centre (k+1)*interval: scaled offset ((k+1) - u)*len_step
                                const float beta_c = ((float)(start + WL / 2 + 1) - u) * bc.len_step;
                                const WindowSeed s = window_seed(beta_c, bc.len_step, w);
                                window_scatter<WL>(myhist + start, s, bc.len_cc);
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
                                        window_scatter<WA>(myhist + (ax + 1) * HS + start, s, bc.ang_cc);
                                    }
                                }
                            }
                        }
                    }
                }
                __syncthreads();
            }

            if (HAS_LEN) {
                // ---- merge the replicas into float bins (and clear them for the next pair)
                for (int u = lane; u < (HAS_ANG ? 4 : 1) * HS; u += WAVE) shat[u] = take_bin(hist, u);
                __syncthreads();
                // ---- projection by this lane's weight row
                float acc = 0.0f;
                const float4* hrow = reinterpret_cast<const float4*>(shat + enc * HS);
                if (HAS_ANG || enc == 0) {
#pragma unroll
                    for (int k4 = 0; k4 < NBINS / 4; k4++) {
                        const float4 hv = hrow[k4];
                        acc = fmaf(Wrow[4 * k4 + 0], hv.x, acc);
                        acc = fmaf(Wrow[4 * k4 + 1], hv.y, acc);
                        acc = fmaf(Wrow[4 * k4 + 2], hv.z, acc);
                        acc = fmaf(Wrow[4 * k4 + 3], hv.w, acc);
                    }
                }
                acc *= enc_coef;
                acc += __shfl_xor(acc, 16, WAVE);
                acc += __shfl_xor(acc, 32, WAVE);
                if (lane < DH) P.out_psi[((size_t)e * H + h) * DH + lane] = acc;
            }
            if (lane == 0) {
                P.out_z[(size_t)e * H + h] = logf(S) + d2min * a;
                if (P.out_d2min) P.out_d2min[(size_t)e * H + h] = d2min;
            }
        }
        if (P.stats && lane == 0) {
            atomicAdd(P.stats + STAT_FWD_EVAL, n_eval);
            atomicAdd(P.stats + STAT_FWD_RAW, (unsigned long long)bx.T * (unsigned long long)(e1 - e0));
            atomicAdd(P.stats + STAT_FWD_PAIRS, (unsigned long long)(e1 - e0));
        }
    }
}

}  // namespace cfh
