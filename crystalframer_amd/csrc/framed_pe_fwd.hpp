// Forward of the framed value position encoding: z, psi (and optionally d2min) for every
// (pair, head).  One launch covers what the reference does in two kernels plus a tensor sum
// (models/kernels/real_enc_frame_proj_fwd_length.cu, ..._fwd_angle.cu,
//  models/cuda_funcs/real_space_framed_proj.py:63-105).
//
// Per (atom i, head h) item, pairs e=(i,j) taken GROUP at a time:
//   per pair, lanes over translations n:
//     pass A  d2min = min_n |r_ij + n.L|^2                                (6 VALU per translation)
//     pass B  w_n = 2^(a'(d^2-d2min)); S = sum_n w_n; the translations with w_n >= 2^-prune are
//             appended (ballot/prefix compaction) to the group's LDS list
//   per group, lanes over the list:
//     pass C  p = w/S; scatter p*g_k(d) into the pair's 9-bin distance window and p*g_m(cos(n,f_axis))
//             into its three 33-bin angle windows (fixed-point LDS adds, Gaussians by recurrence)
//   per pair:
//     epilogue lane (enc,c): psi_enc[c] = W_enc[h,c,:] . hist_enc, W rows held in registers;
//             z = log S + a d2min.
#pragma once
#include "device_common.hpp"

namespace cfh {

template <int WL, int WA, bool COS_ABS, bool HAS_LEN, bool HAS_ANG>
__global__ __launch_bounds__(WAVE) void framed_pe_fwd_kernel(const KernelArgs P) {
    __shared__ float4 tab[TCAP];
    __shared__ uint16_t list[LISTCAP];
    __shared__ uint32_t hist[GROUP * PAIR_STRIDE];
    __shared__ __attribute__((aligned(16))) float shat[4 * HS];
    __shared__ float4 pairA[GROUP];        // rx, ry, rz, d2min of the pairs of the group
    __shared__ float2 pairS[GROUP];        // S and 2^31/S

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

    for (int u = lane; u < GROUP * PAIR_STRIDE; u += WAVE) hist[u] = 0u;
    __syncthreads();

    unsigned long long st_eval = 0, st_raw = 0, st_pairs = 0;
    for (int it = first_item(H); it < P.N; it += item_stride(H)) {
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
        int nlist = 0;

        // pass C over the current list; the table the entries point into must still be resident
        auto flush = [&]() {
            __syncthreads();                       // list and pair data written
            if (HAS_LEN) {
                const int nb = (nlist + WAVE - 1) / WAVE;
                for (int bt = 0; bt < nb; bt++) {
                    const int idx = lane * nb + bt;       // every nb-th entry: lanes spread over the pairs
                    if (idx < nlist) {
                        const uint32_t ent = list[idx];
                        const int el = ent >> (16 - GROUP_BITS);
                        const float4 v = tab[ent & ((1u << (16 - GROUP_BITS)) - 1u)];
                        const float4 pa = pairA[el];
                        const float dx = pa.x + v.x, dy = pa.y + v.y, dz = pa.z + v.z;
                        const float d2 = fmaf(dx, dx, fmaf(dy, dy, dz * dz));
                        const float w = hw_exp2(a2 * (d2 - pa.w)) * pairS[el].y;
                        uint32_t* const myhist = hist + el * PAIR_STRIDE;
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
            n_eval += (unsigned long long)nlist;
            nlist = 0;
            __syncthreads();                       // list may be refilled, histograms may be read
        };

        for (int g0 = e0; g0 < e1; g0 += GROUP) {
            const int ng = min(GROUP, e1 - g0);
            for (int el = 0; el < ng; el++) {
                const int e = g0 + el;
                const float rx = uniform_f(P.rpos[(size_t)e * 3 + 0]);
                const float ry = uniform_f(P.rpos[(size_t)e * 3 + 1]);
                const float rz = uniform_f(P.rpos[(size_t)e * 3 + 2]);

                // ---- pass A: nearest image
                float d2min = 3.0e38f;
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
                    if (lane == 0) {
                        pairA[el] = make_float4(rx, ry, rz, d2min);
                        pairS[el] = make_float2(S, FIX_ONE / S);
                    }
                }

                // ---- pass B: weights, normaliser, compaction of the translations that matter
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
                        if (keep) list[nlist + lane_prefix(m)] = (uint16_t)((el << (16 - GROUP_BITS)) | u);
                        nlist += __popcll(m);
                    }
                    if (nchunks == 1) {
                        S = wave_sum(Sb);
                        if (lane == 0) {
                            pairA[el] = make_float4(rx, ry, rz, d2min);
                            pairS[el] = make_float2(S, FIX_ONE / S);
                        }
                    } else {
                        flush();       // the entries point into this chunk of the table
                    }
                }
            }
            flush();

            // ---- per pair: histogram -> float bins, projection by this lane's weight row, stores
            for (int el = 0; el < ng; el++) {
                const int e = g0 + el;
                if (HAS_LEN) {
                    for (int u = lane; u < (HAS_ANG ? 4 : 1) * HS; u += WAVE)
                        shat[u] = take_bin(hist + el * PAIR_STRIDE, u);
                    __syncthreads();
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
                    __syncthreads();               // shat is rewritten for the next pair
                }
                if (lane == 0) {
                    const float d2min = pairA[el].w;
                    P.out_z[(size_t)e * H + h] = logf(pairS[el].x) + d2min * a;
                    if (P.out_d2min) P.out_d2min[(size_t)e * H + h] = d2min;
                }
            }
            __syncthreads();                       // pair data of this group no longer needed
        }
        st_eval += n_eval;
        st_raw += (unsigned long long)bx.T * (unsigned long long)(e1 - e0);
        st_pairs += (unsigned long long)(e1 - e0);
    }
    // one set of atomics per wavefront (per-item atomics on three shared addresses serialise in L2)
    if (P.stats && lane == 0) {
        atomicAdd(P.stats + STAT_FWD_EVAL, st_eval);
        atomicAdd(P.stats + STAT_FWD_RAW, st_raw);
        atomicAdd(P.stats + STAT_FWD_PAIRS, st_pairs);
    }
}

}  // namespace cfh
