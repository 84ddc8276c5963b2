// Backward of the framed value position encoding: dL/da (N,H) and dL/dW for the four projection
// weights, in one launch plus a small reduction.  Replaces the reference's
// real_enc_frame_proj_bwd_length / real_enc_frame_proj_bwd_angle kernels
// (models/kernels/real_enc_frame_proj_bwd_length.cu:100-237, ..._bwd_angle.cu:104-275) and the
// sums around them (models/cuda_funcs/real_space_framed_proj.py:123-221).
//
// With p_n = exp(a d_n^2 - z) (recomputed, never stored), G_enc[k] = coef_enc sum_c W_enc[h,c,k] gpsi[c]
// and bg_n = sum_enc sum_{k in window} g_k(x_enc,n) G_enc[k]:
//   ga_ih   = sum_j [ gz sum_n p d^2 + sum_n p d^2 bg - (sum_n p d^2)(sum_n p bg) ]
//   gW_enc[h,c,k] = coef_enc sum_e gpsi[e,h,c] sum_n p g_k
// Lane k of the wavefront keeps W_enc[h,:,k] and the running gW_enc[h,:,k] in registers for the
// whole launch; partials are written once per wavefront and summed by gw_reduce_kernel, so no
// global atomics touch the weight gradients.
#pragma once
#include "device_common.hpp"

namespace cfh {

template <int WL, int WA, bool COS_ABS, bool HAS_LEN, bool HAS_ANG>
__global__ __launch_bounds__(WAVE) void framed_pe_bwd_kernel(const KernelArgs P) {
    __shared__ float4 tab[TCAP];
    __shared__ uint16_t list[TCAP];
    __shared__ uint32_t hist[NREP * REP_STRIDE];                  // fixed-point sum_n p g_k per encoder
    __shared__ __attribute__((aligned(16))) float Gs[4 * HS];     // projected upstream gradient / 2^31

    constexpr int NENC = HAS_ANG ? 4 : (HAS_LEN ? 1 : 0);
    const int lane = threadIdx.x;
    const int H = P.H;
    const int h = blockIdx.x % H;
    uint32_t* const myhist = hist + (lane & (NREP - 1)) * REP_STRIDE;

    // lane k: W_enc[h, c, k] for all (enc, c), and the gradient accumulators of the same shape
    float Wt[NENC > 0 ? NENC * DH : 1];
    float gW[NENC > 0 ? NENC * DH : 1];
#pragma unroll
    for (int en = 0; en < NENC; en++)
#pragma unroll
        for (int c = 0; c < DH; c++) {
            Wt[en * DH + c] = P.W[en][((size_t)h * DH + c) * NBINS + lane];
            gW[en * DH + c] = 0.0f;
        }
    const BasisConsts bc = P.bc;
    const float prune = (P.prune_log2 > 0.0f) ? -P.prune_log2 : -3.0e38f;

    for (int u = lane; u < NREP * REP_STRIDE; u += WAVE) hist[u] = 0u;
    for (int u = lane; u < 4 * HS; u += WAVE) Gs[u] = 0.0f;
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
        float ga_acc = 0.0f;
        unsigned long long n_eval = 0;

        for (int e = e0; e < e1; e++) {
            const float rx = uniform_f(P.rpos[(size_t)e * 3 + 0]);
            const float ry = uniform_f(P.rpos[(size_t)e * 3 + 1]);
            const float rz = uniform_f(P.rpos[(size_t)e * 3 + 2]);
            const float z2 = uniform_f(P.z[(size_t)e * H + h]) * LOG2E;
            const float gz = uniform_f(P.gz[(size_t)e * H + h]);

            // upstream gradient of psi, projected onto the bins:  G_enc[k] (this lane: k = lane)
            float gp[DH];
            if (NENC > 0) {
#pragma unroll
                for (int c = 0; c < DH; c++) gp[c] = uniform_f(P.gpsi[((size_t)e * H + h) * DH + c]);
            }
            __syncthreads();       // previous pair's reads of Gs are done
#pragma unroll
            for (int en = 0; en < NENC; en++) {
                float g = 0.0f;
#pragma unroll
                for (int c = 0; c < DH; c++) g = fmaf(Wt[en * DH + c], gp[c], g);
                Gs[en * HS + lane] = g * ((en == 0 ? P.dist_coef : P.angle_coef) * FIX_INV);
            }
            __syncthreads();

            float A0 = 0.0f, A1 = 0.0f, A2 = 0.0f;   // sum p d^2, sum p d^2 bg, sum p bg
            for (int ch = 0; ch < nchunks; ch++) {
                const int t0 = ch * TCAP;
                const int cnt = min(TCAP, bx.T - t0);
                if (nchunks > 1) {
                    __syncthreads();
                    build_shift_table(tab, t0, cnt, bx, L, lane);
                    __syncthreads();
                }
                int nkeep = 0;
                for (int u0 = 0; u0 < cnt; u0 += WAVE) {
                    const int u = u0 + lane;
                    bool keep = false;
                    if (u < cnt) {
                        const float4 v = tab[u];
                        const float dx = rx + v.x, dy = ry + v.y, dz = rz + v.z;
                        const float d2 = fmaf(dx, dx, fmaf(dy, dy, dz * dz));
                        const float ex = fmaf(a2, d2, -z2);
                        keep = ex >= prune;
                        if (!keep) A0 = fmaf(hw_exp2(ex), d2, A0);    // light terms still count in dz/da
                    }
                    const uint64_t m = __ballot(keep);
                    if (keep) list[nkeep + lane_prefix(m)] = (uint16_t)u;
                    nkeep += __popcll(m);
                }
                n_eval += (unsigned long long)nkeep;
                __syncthreads();
                for (int v0 = 0; v0 < nkeep; v0 += WAVE) {
                    if (v0 + lane < nkeep) {
                        const float4 v = tab[list[v0 + lane]];
                        const float dx = rx + v.x, dy = ry + v.y, dz = rz + v.z;
                        const float d2 = fmaf(dx, dx, fmaf(dy, dy, dz * dz));
                        const float p = hw_exp2(fmaf(a2, d2, -z2));
                        const float pf = p * FIX_ONE;
                        float pbg = 0.0f;
                        if (HAS_LEN) {
                            const float d = hw_sqrt(d2);
                            const float u = d * bc.inv_interval;
                            int start = (int)(u - bc.start_off);
                            start = max(0, min(start, NBINS - WL));
                            const float beta_c = ((float)(start + WL / 2 + 1) - u) * bc.len_step;
                            const WindowSeed s = window_seed(beta_c, bc.len_step, pf);
                            pbg += window_scatter_gather<WL>(myhist + start, Gs + start, s, bc.len_cc);
                        }
                        if (HAS_ANG) {
                            if (d2 > 1e-5f) {
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
                                    const WindowSeed s = window_seed(beta_c, bc.ang_step, pf);
                                    pbg += window_scatter_gather<WA>(myhist + (ax + 1) * HS + start,
                                                                     Gs + (ax + 1) * HS + start, s, bc.ang_cc);
                                }
                            }
                        }
                        A0 = fmaf(p, d2, A0);
                        A1 = fmaf(d2, pbg, A1);
                        A2 += pbg;
                    }
                }
                __syncthreads();
            }
            A0 = wave_sum(A0); A1 = wave_sum(A1); A2 = wave_sum(A2);
            ga_acc += P.gz_coef * gz * A0 + (A1 - A0 * A2);

            // weight gradients: gW_enc[c] (lane k) += coef * gpsi[c] * s_enc[k]
#pragma unroll
            for (int en = 0; en < NENC; en++) {
                const float sk = take_bin(hist, en * HS + lane) * (en == 0 ? P.gw_dist_coef : P.angle_coef);
#pragma unroll
                for (int c = 0; c < DH; c++) gW[en * DH + c] = fmaf(gp[c], sk, gW[en * DH + c]);
            }
        }
        if (lane == 0) {
            P.out_ga[(size_t)i * H + h] = ga_acc;
            if (P.stats) {
                atomicAdd(P.stats + STAT_BWD_EVAL, n_eval);
                atomicAdd(P.stats + STAT_BWD_RAW, (unsigned long long)bx.T * (unsigned long long)(e1 - e0));
                atomicAdd(P.stats + STAT_BWD_PAIRS, (unsigned long long)(e1 - e0));
            }
        }
    }

    // per-wavefront partials of the weight gradients: (wave, enc, c, k)
    if (NENC > 0) {
        float* dst = P.gw_partial + (size_t)blockIdx.x * 4 * DH * NBINS;
#pragma unroll
        for (int en = 0; en < NENC; en++)
#pragma unroll
            for (int c = 0; c < DH; c++) dst[(en * DH + c) * NBINS + lane] = gW[en * DH + c];
    }
}

// gW_enc[h, c, k] = sum over the wavefronts w of head h (w % H == h) of partial[w, enc, c, k].
__global__ __launch_bounds__(256) void gw_reduce_kernel(const float* __restrict__ partial, int nwaves,
                                                        int H, int nenc, float* out0, float* out1,
                                                        float* out2, float* out3) {
    const int idx = blockIdx.x * blockDim.x + threadIdx.x;       // over (enc, h, c, k)
    const int per_enc = H * DH * NBINS;
    if (idx >= nenc * per_enc) return;
    const int en = idx / per_enc;
    const int rem = idx % per_enc;
    const int h = rem / (DH * NBINS);
    const int ck = rem % (DH * NBINS);
    float s = 0.0f;
    for (int w = h; w < nwaves; w += H) s += partial[((size_t)w * 4 + en) * DH * NBINS + ck];
    float* out = en == 0 ? out0 : (en == 1 ? out1 : (en == 2 ? out2 : out3));
    if (out) out[rem] = s;
}

}  // namespace cfh
