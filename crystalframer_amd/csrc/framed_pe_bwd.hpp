// Backward of the framed value position encoding: dL/da (N,H) and dL/dW for the four projection
// weights, in one launch plus a small reduction.  Replaces the reference's
// real_enc_frame_proj_bwd_length / real_enc_frame_proj_bwd_angle kernels
// (models/kernels/real_enc_frame_proj_bwd_length.cu:100-237, ..._bwd_angle.cu:104-275) and the
// sums around them (models/cuda_funcs/real_space_framed_proj.py:123-221).
//
// With p_n = exp(a d_n^2 - z) (recomputed, never stored), G_enc[k] = coef_enc sum_c W_enc[h,c,k] gpsi[c],
// bg_n = sum_enc sum_{k in window} g_k(x_enc,n) G_enc[k] and A0 = sum_n p_n d_n^2:
//   ga_ih   = sum_j [ gz A0 + sum_n p_n (d_n^2 - A0) bg_n ]          (the reference's covariance form
//             sum p d^2 bg - (sum p d^2)(sum p bg), written without the cancellation)
//   gW_enc[h,c,k] = coef_enc sum_e gpsi[e,h,c] sum_n p g_k
// Pairs are taken GROUP_BWD at a time: per pair a light sweep gives A0 and compacts the translations
// that matter into the group's list, the heavy pass (window gather + scatter) runs over the list with
// full lanes.  Lane k of the wavefront keeps W_enc[h,:,k] and the running gW_enc[h,:,k] in registers
// for the whole launch; partials are written once per wavefront and summed by gw_reduce_kernel, so no
// global atomics touch the weight gradients.
#pragma once
#include "device_common.hpp"

namespace cfh {

template <int WL, int WA, bool COS_ABS, bool HAS_LEN, bool HAS_ANG>
__global__ __launch_bounds__(WAVE) void framed_pe_bwd_kernel(const KernelArgs P) {
    __shared__ float4 tab[TCAP];
    __shared__ uint16_t list[LISTCAP];
    __shared__ uint32_t hist[GROUP_BWD * PAIR_STRIDE];                              // fixed-point sum_n p g_k
    __shared__ __attribute__((aligned(16))) float Gs[GROUP_BWD * PAIR_STRIDE];      // G / 2^31 per pair
    __shared__ __attribute__((aligned(16))) float gpS[GROUP_BWD * DH];              // gpsi of the pairs
    __shared__ float4 pairA[GROUP_BWD];     // rx, ry, rz, A0
    __shared__ float pairZ[GROUP_BWD];      // z * log2(e)

    constexpr int NENC = HAS_ANG ? 4 : (HAS_LEN ? 1 : 0);
    const int lane = threadIdx.x;
    const int H = P.H;
    const int h = blockIdx.x % H;

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

    for (int u = lane; u < GROUP_BWD * PAIR_STRIDE; u += WAVE) { hist[u] = 0u; Gs[u] = 0.0f; }
    __syncthreads();

    unsigned long long st_eval = 0, st_raw = 0, st_pairs = 0;
    // software pipeline over items: record of item n+1 and queue ticket of item n+2 in flight
    int queue = first_queue(H);
    int it_cur = queue_pop(P, h, queue);
    int it_next = it_cur >= 0 ? queue_pop(P, h, queue) : -1;
    uint32_t rec_cur = load_record(P, it_cur, h);
    while (it_cur >= 0) {
        const int ticket = queue_ticket(P, h, queue);
        const uint32_t rec_next = load_record(P, it_next, h);
        const Item item = unpack_item(rec_cur);
        const int i = item.i;
        const float a = item.a;
        const float a2 = a * LOG2E;
        const Lattice L = item.L;
        const Box bx = item.bx;
        float f[3][3];
        if (HAS_ANG) {
#pragma unroll
            for (int ax = 0; ax < 3; ax++)
#pragma unroll
                for (int d = 0; d < 3; d++) f[ax][d] = rec_f(rec_cur, REC_FRAMES + ax * 3 + d);
        }
        const int nchunks = (bx.T + TCAP - 1) / TCAP;
        if (nchunks == 1) {
            __syncthreads();
            build_shift_table(tab, 0, bx.T, bx, L, lane);
            __syncthreads();
        }
        const int e0 = item.e0;
        const int e1 = e0 + item.npairs;
        float ga_acc = 0.0f;      // uniform part: sum_e gz A0
        float cov = 0.0f;         // per lane: sum over its terms of p (d^2 - A0) bg
        unsigned long long n_eval = 0;
        int nlist = 0;

        // heavy pass over the current list; the table the entries point into must still be resident
        auto flush = [&]() {
            __syncthreads();
            if (NENC > 0) {
                const int nb = (nlist + WAVE - 1) / WAVE;
                for (int bt = 0; bt < nb; bt++) {
                    const int idx = lane * nb + bt;
                    if (idx < nlist) {
                        const uint32_t ent = list[idx];
                        const int el = ent >> (16 - GROUP_BITS);
                        const float4 v = tab[ent & ((1u << (16 - GROUP_BITS)) - 1u)];
                        const float4 pa = pairA[el];
                        const float dx = pa.x + v.x, dy = pa.y + v.y, dz = pa.z + v.z;
                        const float d2 = fmaf(dx, dx, fmaf(dy, dy, dz * dz));
                        const float pf = hw_exp2(fmaf(a2, d2, -pairZ[el])) * FIX_ONE;
                        uint32_t* const myhist = hist + el * PAIR_STRIDE;
                        const float* const myG = Gs + el * PAIR_STRIDE;
                        float pbg = 0.0f;
                        {
                            const float d = hw_sqrt(d2);
                            const float u = d * bc.inv_interval;
                            int start = (int)(u - bc.start_off);
                            start = max(0, min(start, NBINS - WL));
                            const float beta_c = ((float)(start + WL / 2 + 1) - u) * bc.len_step;
                            const WindowSeed s = window_seed(beta_c, bc.len_step, pf);
                            pbg += window_scatter_gather<WL>(myhist + start, myG + start, s, bc.len_cc);
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
                                                                     myG + (ax + 1) * HS + start, s, bc.ang_cc);
                                }
                            }
                        }
                        cov = fmaf(d2 - pa.w, pbg, cov);
                    }
                }
            }
            n_eval += (unsigned long long)nlist;
            nlist = 0;
            __syncthreads();
        };

        for (int g0 = e0; g0 < e1; g0 += GROUP_BWD) {
            const int ng = min(GROUP_BWD, e1 - g0);
            // stage gpsi of the group's pairs (coalesced: 16 consecutive floats per pair)
            if (NENC > 0 && lane < ng * DH) gpS[lane] = P.gpsi[((size_t)g0 * H) * DH + (size_t)(lane / DH) * H * DH + (size_t)h * DH + (lane % DH)];
            __syncthreads();

            for (int el = 0; el < ng; el++) {
                const int e = g0 + el;
                const float rx = uniform_f(P.rpos[(size_t)e * 3 + 0]);
                const float ry = uniform_f(P.rpos[(size_t)e * 3 + 1]);
                const float rz = uniform_f(P.rpos[(size_t)e * 3 + 2]);
                const float z2 = uniform_f(P.z[(size_t)e * H + h]) * LOG2E;
                const float gz = uniform_f(P.gz[(size_t)e * H + h]);

                // upstream gradient of psi projected onto the bins: G_enc[k], this lane: k = lane
                if (NENC > 0) {
                    float gp[DH];
#pragma unroll
                    for (int c4 = 0; c4 < DH / 4; c4++) {
                        const float4 t4 = reinterpret_cast<const float4*>(gpS + el * DH)[c4];
                        gp[4 * c4 + 0] = t4.x; gp[4 * c4 + 1] = t4.y; gp[4 * c4 + 2] = t4.z; gp[4 * c4 + 3] = t4.w;
                    }
#pragma unroll
                    for (int en = 0; en < NENC; en++) {
                        float g = 0.0f;
#pragma unroll
                        for (int c = 0; c < DH; c++) g = fmaf(Wt[en * DH + c], gp[c], g);
                        Gs[el * PAIR_STRIDE + en * HS + lane] = g * ((en == 0 ? P.dist_coef : P.angle_coef) * FIX_INV);
                    }
                }

                // light sweep: A0 = sum_n p d^2 over every translation, compaction of those that matter
                float A0 = 0.0f;
                for (int ch = 0; ch < nchunks; ch++) {
                    const int t0 = ch * TCAP;
                    const int cnt = min(TCAP, bx.T - t0);
                    if (nchunks > 1) {
                        flush();
                        build_shift_table(tab, t0, cnt, bx, L, lane);
                        __syncthreads();
                    }
                    for (int u = lane; u < cnt; u += WAVE) {
                        const float4 v = tab[u];
                        const float dx = rx + v.x, dy = ry + v.y, dz = rz + v.z;
                        const float d2 = fmaf(dx, dx, fmaf(dy, dy, dz * dz));
                        A0 = fmaf(hw_exp2(fmaf(a2, d2, -z2)), d2, A0);
                    }
                }
                A0 = wave_sum(A0);
                ga_acc = fmaf(P.gz_coef * gz, A0, ga_acc);
                if (lane == 0) {
                    pairA[el] = make_float4(rx, ry, rz, A0);
                    pairZ[el] = z2;
                }
                for (int ch = 0; ch < nchunks; ch++) {
                    const int t0 = ch * TCAP;
                    const int cnt = min(TCAP, bx.T - t0);
                    if (nchunks > 1) {
                        __syncthreads();
                        build_shift_table(tab, t0, cnt, bx, L, lane);
                        __syncthreads();
                    } else if (nlist + cnt > LISTCAP) {
                        flush();
                    }
                    for (int u0 = 0; u0 < cnt; u0 += WAVE) {
                        const int u = u0 + lane;
                        bool keep = false;
                        if (u < cnt) {
                            const float4 v = tab[u];
                            const float dx = rx + v.x, dy = ry + v.y, dz = rz + v.z;
                            keep = fmaf(a2, fmaf(dx, dx, fmaf(dy, dy, dz * dz)), -z2) >= prune;
                        }
                        const uint64_t m = __ballot(keep);
                        if (keep) list[nlist + lane_prefix(m)] = (uint16_t)((el << (16 - GROUP_BITS)) | u);
                        nlist += __popcll(m);
                    }
                    if (nchunks > 1) flush();
                }
            }
            flush();

            // weight gradients: gW_enc[c] (lane k) += coef * gpsi[c] * s_enc[k]
            if (NENC > 0) {
                for (int el = 0; el < ng; el++) {
                    float gp[DH];
#pragma unroll
                    for (int c4 = 0; c4 < DH / 4; c4++) {
                        const float4 t4 = reinterpret_cast<const float4*>(gpS + el * DH)[c4];
                        gp[4 * c4 + 0] = t4.x; gp[4 * c4 + 1] = t4.y; gp[4 * c4 + 2] = t4.z; gp[4 * c4 + 3] = t4.w;
                    }
#pragma unroll
                    for (int en = 0; en < NENC; en++) {
                        const float sk = take_bin(hist + el * PAIR_STRIDE, en * HS + lane) *
                                         (en == 0 ? P.gw_dist_coef : P.angle_coef);
#pragma unroll
                        for (int c = 0; c < DH; c++) gW[en * DH + c] = fmaf(gp[c], sk, gW[en * DH + c]);
                    }
                }
            }
            __syncthreads();               // gpS, pair data and histograms are free again
        }
        cov = wave_sum(cov);
        if (lane == 0) P.out_ga[(size_t)i * H + h] = ga_acc + cov;
        st_eval += n_eval;
        st_raw += (unsigned long long)bx.T * (unsigned long long)(e1 - e0);
        st_pairs += (unsigned long long)(e1 - e0);
        it_cur = it_next;
        rec_cur = rec_next;
        it_next = it_cur >= 0 ? queue_redeem(P, h, queue, ticket) : -1;
    }
    if (P.stats && lane == 0) {      // once per wavefront
        atomicAdd(P.stats + STAT_BWD_EVAL, st_eval);
        atomicAdd(P.stats + STAT_BWD_RAW, st_raw);
        atomicAdd(P.stats + STAT_BWD_PAIRS, st_pairs);
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

// gW_enc[h, c, k] += sum over a slice of the wavefronts w of head h (w % H == h) of
// partial[w, enc, c, k]; the outputs are cleared by zero_outputs_kernel first.
__global__ __launch_bounds__(256) void gw_reduce_kernel(const float* __restrict__ partial, int nwaves,
                                                        int H, int nenc, int nslices, float* out0,
                                                        float* out1, float* out2, float* out3) {
    const int idx = blockIdx.x * blockDim.x + threadIdx.x;       // over (enc, h, c, k)
    const int per_enc = H * DH * NBINS;
    if (idx >= nenc * per_enc) return;
    const int en = idx / per_enc;
    const int rem = idx % per_enc;
    const int h = rem / (DH * NBINS);
    const int ck = rem % (DH * NBINS);
    float s = 0.0f;
    for (int w = h + H * blockIdx.y; w < nwaves; w += H * nslices)
        s += partial[((size_t)w * 4 + en) * DH * NBINS + ck];
    float* out = en == 0 ? out0 : (en == 1 ? out1 : (en == 2 ? out2 : out3));
    if (out) atomicAdd(out + rem, s);
}

__global__ __launch_bounds__(256) void zero_outputs_kernel(int n, float* out0, float* out1, float* out2,
                                                           float* out3) {
    const int idx = blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= n) return;
    if (out0) out0[idx] = 0.0f;
    if (out1) out1[idx] = 0.0f;
    if (out2) out2[idx] = 0.0f;
    if (out3) out3[idx] = 0.0f;
}

}  // namespace cfh
