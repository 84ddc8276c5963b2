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
//
// Pairs are taken 4 at a time, one per 16-lane row:
//   G of the 4 pairs: 64 MFMA 4x4x1 steps -- lane k holds W_enc[h,:,k] in registers for the whole
//     launch (A operand: block = k/4), the B operand is gpsi[pair = lane%4][c]; result to LDS;
//   light sweep (rows over the translations): A0, compaction of the translations that matter into
//     the group's list;
//   heavy pass over the list with full lanes: window gather from G, window scatter of p g_k into
//     the pair's fixed-point histogram;
//   weight gradients: 64 MFMA 4x4x1 steps per 4 pairs, A = the histogram bin k of a pair,
//     B = gpsi[pair][4 cq + lane%4]; the 16 accumulators (enc, cq) stay in registers for the whole
//     launch and are written once per wavefront, summed by gw_reduce_kernel, so no global atomics
//     touch the weight gradients.
#pragma once
#include "device_common.hpp"

namespace cfh {

constexpr int BWD_TCAP = 256;          // translations staged in LDS at a time (4 KB)
constexpr int BWD_LISTCAP = 512;       // entries of the survivor list (a round that overflows it is repeated)
constexpr int BWD_SHIFT = 13;          // list entry = pair-in-group << 13 | table index
static_assert(GROUP_BWD == 4, "one pair per 16-lane row, 4 pairs per MFMA column set");

typedef float v4f_b __attribute__((ext_vector_type(4)));

template <int WL, int WA, bool COS_ABS, bool HAS_LEN, bool HAS_ANG>
__global__ __launch_bounds__(WAVE) void framed_pe_bwd_kernel(const KernelArgs P) {
    __shared__ float4 tab[BWD_TCAP];
    __shared__ uint16_t list[BWD_LISTCAP];
    __shared__ __attribute__((aligned(16))) uint32_t hist[GROUP_BWD * PAIR_STRIDE];   // fixed-point sum_n p g_k
    __shared__ __attribute__((aligned(16))) float Gs[GROUP_BWD * PAIR_STRIDE];        // G / 2^31 per pair
    __shared__ __attribute__((aligned(16))) float gpS[GROUP_BWD * DH];     // gpsi[p][c]
    __shared__ __attribute__((aligned(16))) float gpT[GROUP_BWD * DH];     // gpsi[p][c] at (p*4 + c%4)*4 + c/4
    __shared__ float4 pairA[GROUP_BWD];     // rx, ry, rz, A0
    __shared__ float pairZ[GROUP_BWD];      // z * log2(e)

    constexpr int NENC = HAS_ANG ? 4 : (HAS_LEN ? 1 : 0);
    const int lane = threadIdx.x;
    const int H = P.H;
    const int h = blockIdx.x % H;
    const int slot = lane >> 4;       // light sweep: which pair of the group
    const int tl = lane & 15;         // light sweep: position in the row
    const int sub = lane & 3;         // MFMA column (B operand, result) of this lane
    const int blk = lane >> 2;        // MFMA block of this lane

    // lane k: W_enc[h, c, k] for all (enc, c); accumulators of the weight gradients
    float Wt[NENC > 0 ? NENC * DH : 1];
    v4f_b gWacc[NENC > 0 ? NENC * 4 : 1];
#pragma unroll
    for (int en = 0; en < NENC; en++) {
#pragma unroll
        for (int c = 0; c < DH; c++) Wt[en * DH + c] = P.W[en][((size_t)h * DH + c) * NBINS + lane];
#pragma unroll
        for (int cq = 0; cq < 4; cq++) gWacc[en * 4 + cq] = v4f_b{0.f, 0.f, 0.f, 0.f};
    }
    const BasisConsts bc = P.bc;
    const int WLr = WL > 0 ? WL : bc.len_window;      // bins of the distance window (WL == 0: known at run time only)
    const float prune = (P.prune_log2 > 0.0f) ? -P.prune_log2 : -3.0e38f;

    for (int u = lane; u < GROUP_BWD * PAIR_STRIDE; u += WAVE) { hist[u] = 0u; Gs[u] = 0.0f; }
    wave_sync();

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
        const float a2 = item.a * LOG2E;
        const Lattice L = item.L;
        const Box bx = item.bx;
        float f[3][3];
        if (HAS_ANG) {
#pragma unroll
            for (int ax = 0; ax < 3; ax++)
#pragma unroll
                for (int d = 0; d < 3; d++) f[ax][d] = rec_f(rec_cur, REC_FRAMES + ax * 3 + d);
        }
        const int nchunks = (bx.T + BWD_TCAP - 1) / BWD_TCAP;
        if (nchunks == 1) {
            wave_sync();
            build_shift_table(tab, 0, bx.T, bx, L, lane);
            wave_sync();
        }
        const int e0 = item.e0;
        const int npairs = item.npairs;
        const int e1 = e0 + npairs;
        float cov = 0.0f;         // per lane: its share of sum_e [gz A0 + sum_n p (d^2 - A0) bg]
        unsigned long long n_eval = 0;
        int nlist = 0;

        // ---- heavy pass over the current list; the table the entries point into is still resident
        auto flush = [&]() {
            wave_sync();
            if (NENC > 0) {
                const int nb = (nlist + WAVE - 1) / WAVE;
                for (int bt = 0; bt < nb; bt++) {
                    const int idx = (((lane & 15) << 2) | (lane >> 4)) * nb + bt;   // neighbours in different rows, as in the forward
                    if (idx < nlist) {
                        const uint32_t ent = list[idx];
                        const int el = ent >> BWD_SHIFT;
                        const float4 v = tab[ent & ((1u << BWD_SHIFT) - 1u)];
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
                            start = max(0, min(start, NBINS - WLr));
                            const float beta_c = ((float)(start + WLr / 2 + 1) - u) * bc.len_step;
                            const WindowSeed s = window_seed(beta_c, bc.len_step, pf);
                            pbg += window_scatter_gather<WL>(myhist + start, myG + start, s, bc.len_cc, WLr);
                        }
                        if (HAS_ANG) {
                            if (d2 > 1e-5f) {
                                const float rinv = hw_rsq(d2);
#pragma unroll
                                for (int ax = 0; ax < 3; ax++) {
                                    float cs = (dx * f[ax][0] + dy * f[ax][1] + dz * f[ax][2]) * rinv;
                                    if (COS_ABS) cs = fabsf(cs);
                                    int end = (int)fminf((cs + bc.ang_end_off) * bc.ang_inv_interval + 1.0f,
                                                         bc.ang_end_max);
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
            wave_sync();
        };

        // ---- weight gradients of the ng pairs of the finished group; clears their histograms
        auto gw_update = [&](int ng) {
            if (NENC > 0) {
                for (int p = 0; p < ng; p++) {
                    const float4 gq = reinterpret_cast<const float4*>(gpT)[p * 4 + sub];   // gpsi[p][4 cq + sub]
#pragma unroll
                    for (int en = 0; en < NENC; en++) {
                        uint32_t* hb = hist + p * PAIR_STRIDE + en * HS + lane;
                        const float sk = (float)(*hb);
                        *hb = 0u;
                        gWacc[en * 4 + 0] = __builtin_amdgcn_mfma_f32_4x4x1f32(sk, gq.x, gWacc[en * 4 + 0], 0, 0, 0);
                        gWacc[en * 4 + 1] = __builtin_amdgcn_mfma_f32_4x4x1f32(sk, gq.y, gWacc[en * 4 + 1], 0, 0, 0);
                        gWacc[en * 4 + 2] = __builtin_amdgcn_mfma_f32_4x4x1f32(sk, gq.z, gWacc[en * 4 + 2], 0, 0, 0);
                        gWacc[en * 4 + 3] = __builtin_amdgcn_mfma_f32_4x4x1f32(sk, gq.w, gWacc[en * 4 + 3], 0, 0, 0);
                    }
                }
            }
            wave_sync();               // gpS/gpT, pair data and histograms are free again
        };

        // ---- rounds: group of 4 pairs (one per row), chunk ch of the translations
        float prx = 0.f, pry = 0.f, prz = 0.f, pz2 = 0.f, pgz = 0.f;   // pair (row base + lane)
        float4 pgp = make_float4(0.f, 0.f, 0.f, 0.f);                  // gpsi of pair (block base + lane/4), channels 4 (lane%4)..
        float rx = 0.f, ry = 0.f, rz = 0.f, z2 = 0.f, gzr = 0.f, A0 = 0.f;
        int cur_g0 = -1, cur_ng = 0;
        int el_glob = 0, ch = 0;
        int skip = 0;          // survivors of the current round already processed (list overflow)
        while (true) {
            const bool done = el_glob >= npairs;
            const int g0n = done ? -2 : e0 + el_glob;
            const bool group_change = g0n != cur_g0;
            if (nlist > 0 && (group_change || nchunks > 1 || skip > 0)) flush();
            if (group_change && cur_g0 >= 0) gw_update(cur_ng);
            if (done) break;
            const int el = slot;                           // pair-in-group of this row of lanes
            if (group_change) {
                cur_g0 = g0n;
                cur_ng = min(GROUP_BWD, e1 - g0n);
                if ((el_glob & (WAVE - 1)) == 0) {         // next 64 pairs of the row
                    const int e = e0 + el_glob + lane;
                    if (e < e1) {
                        prx = P.rpos[(size_t)e * 3 + 0];
                        pry = P.rpos[(size_t)e * 3 + 1];
                        prz = P.rpos[(size_t)e * 3 + 2];
                        pz2 = P.z[(size_t)e * H + h] * LOG2E;
                        pgz = P.gz[(size_t)e * H + h];
                    }
                }
                if (NENC > 0) {
                    if ((el_glob & 15) == 0) {             // gpsi of the next 16 pairs: 64 B per pair
                        const int e = e0 + el_glob + (lane >> 2);
                        if (e < e1)
                            pgp = reinterpret_cast<const float4*>(P.gpsi + ((size_t)e * H + h) * DH)[sub];
                    }
                    // the 16 lanes that hold this group's gpsi stage it in both layouts
                    if (((lane >> 4) << 2) == (el_glob & 15)) {
                        const int p = (lane >> 2) & 3;
                        reinterpret_cast<float4*>(gpS)[p * 4 + sub] = pgp;
                        gpT[(p * 4 + 0) * 4 + sub] = pgp.x;
                        gpT[(p * 4 + 1) * 4 + sub] = pgp.y;
                        gpT[(p * 4 + 2) * 4 + sub] = pgp.z;
                        gpT[(p * 4 + 3) * 4 + sub] = pgp.w;
                    }
                    wave_sync();
                    // G[pair = sub][enc][k = 4 blk + r] = sum_c W_enc[c][k] gpsi[pair][c]
                    float gb[DH];
#pragma unroll
                    for (int c4 = 0; c4 < DH / 4; c4++) {
                        const float4 t4 = reinterpret_cast<const float4*>(gpS)[sub * 4 + c4];
                        gb[4 * c4 + 0] = t4.x; gb[4 * c4 + 1] = t4.y; gb[4 * c4 + 2] = t4.z; gb[4 * c4 + 3] = t4.w;
                    }
                    v4f_b g[NENC > 0 ? NENC : 1];
#pragma unroll
                    for (int en = 0; en < NENC; en++) g[en] = v4f_b{0.f, 0.f, 0.f, 0.f};
#pragma unroll
                    for (int c = 0; c < DH; c++)
#pragma unroll
                        for (int en = 0; en < NENC; en++)
                            g[en] = __builtin_amdgcn_mfma_f32_4x4x1f32(Wt[en * DH + c], gb[c], g[en], 0, 0, 0);
#pragma unroll
                    for (int en = 0; en < NENC; en++) {
                        const float sc = (en == 0 ? P.dist_coef : P.angle_coef) * FIX_INV;
                        *reinterpret_cast<float4*>(Gs + sub * PAIR_STRIDE + en * HS + 4 * blk) =
                            make_float4(g[en][0] * sc, g[en][1] * sc, g[en][2] * sc, g[en][3] * sc);
                    }
                }
            }
            const bool active = el < cur_ng;

            if (ch == 0) {
                const int src = (el_glob & (WAVE - 1)) + slot;      // el_glob is a multiple of 4: src <= 63
                rx = __shfl(prx, src, WAVE);
                ry = __shfl(pry, src, WAVE);
                rz = __shfl(prz, src, WAVE);
                z2 = __shfl(pz2, src, WAVE);
                gzr = __shfl(pgz, src, WAVE);
                if (nchunks > 1) {          // A0 over every chunk first: the heavy pass needs it
                    float Ap = 0.0f;
                    for (int cc = 0; cc < nchunks; cc++) {
                        const int t0 = cc * BWD_TCAP;
                        const int cnt = min(BWD_TCAP, bx.T - t0);
                        wave_sync();
                        build_shift_table(tab, t0, cnt, bx, L, lane);
                        wave_sync();
                        for (int u = tl; u < cnt; u += 16) {
                            const float4 v = tab[u];
                            const float dx = rx + v.x, dy = ry + v.y, dz = rz + v.z;
                            const float d2 = fmaf(dx, dx, fmaf(dy, dy, dz * dz));
                            Ap = fmaf(hw_exp2(fmaf(a2, d2, -z2)), d2, Ap);
                        }
                    }
                    A0 = row_sum(Ap);
                    if (active && tl == 0) {
                        pairA[el] = make_float4(rx, ry, rz, A0);
                        pairZ[el] = z2;
                    }
                }
            }

            // ---- light sweep on chunk ch: A0 (single-chunk tables) and compaction
            {
                const int t0 = ch * BWD_TCAP;
                const int cnt = min(BWD_TCAP, bx.T - t0);
                if (nchunks > 1) {
                    wave_sync();
                    build_shift_table(tab, t0, cnt, bx, L, lane);
                    wave_sync();
                }
                float Ap = 0.0f;
                const int room = BWD_LISTCAP - nlist;
                int seen = 0;
                if (bx.T <= 128) {
                    // one slab of 8 translations per lane: all table reads are issued before the arithmetic
                    float d2r[8];
#pragma unroll
                    for (int k = 0; k < 8; k++) {
                        const float4 v = tab[tl + 16 * k];       // beyond T: stale words, masked below
                        const float dx = rx + v.x, dy = ry + v.y, dz = rz + v.z;
                        d2r[k] = fmaf(dx, dx, fmaf(dy, dy, dz * dz));
                    }
#pragma unroll
                    for (int k = 0; k < 8; k++) {
                        const int u = tl + 16 * k;
                        const bool valid = active && u < cnt;
                        const float ex = fmaf(a2, d2r[k], -z2);
                        Ap += valid ? hw_exp2(ex) * d2r[k] : 0.0f;
                        const bool keep = valid && ex >= prune;
                        const uint64_t m = __ballot(keep);
                        const int pos = seen + lane_prefix(m) - skip;
                        if (keep && pos >= 0 && pos < room) list[nlist + pos] = (uint16_t)((el << BWD_SHIFT) | u);
                        seen += __popcll(m);
                    }
                } else {
                    for (int u0 = 0; u0 < cnt; u0 += 16) {
                        const int u = u0 + tl;
                        bool keep = false;
                        if (active && u < cnt) {
                            const float4 v = tab[u];
                            const float dx = rx + v.x, dy = ry + v.y, dz = rz + v.z;
                            const float d2 = fmaf(dx, dx, fmaf(dy, dy, dz * dz));
                            const float ex = fmaf(a2, d2, -z2);
                            if (nchunks == 1) Ap = fmaf(hw_exp2(ex), d2, Ap);
                            keep = ex >= prune;
                        }
                        const uint64_t m = __ballot(keep);
                        const int pos = seen + lane_prefix(m) - skip;
                        if (keep && pos >= 0 && pos < room) list[nlist + pos] = (uint16_t)((el << BWD_SHIFT) | u);
                        seen += __popcll(m);
                    }
                }
                const int appended = min(seen - skip, room);
                nlist += appended;
                skip = (skip + appended < seen) ? skip + appended : 0;   // > 0: repeat the round after a flush
                if (nchunks == 1) {
                    A0 = row_sum(Ap);
                    if (active && tl == 0) {
                        pairA[el] = make_float4(rx, ry, rz, A0);
                        pairZ[el] = z2;
                    }
                }
            }
            if (skip == 0 && ++ch == nchunks) {
                ch = 0;
                el_glob += GROUP_BWD;
                if (active && tl == 0) cov = fmaf(P.gz_coef * gzr, A0, cov);
            }
        }
        cov = wave_sum(cov);
        if (lane == 0) P.out_ga[(size_t)i * H + h] = cov;
        st_eval += n_eval;
        st_raw += (unsigned long long)bx.T * (unsigned long long)npairs;
        st_pairs += (unsigned long long)npairs;
        it_cur = it_next;
        rec_cur = rec_next;
        it_next = it_cur >= 0 ? queue_redeem(P, h, queue, ticket) : -1;
    }
    if (P.stats && lane == 0) {      // once per wavefront
        atomicAdd(P.stats + STAT_BWD_EVAL, st_eval);
        atomicAdd(P.stats + STAT_BWD_RAW, st_raw);
        atomicAdd(P.stats + STAT_BWD_PAIRS, st_pairs);
    }

    // per-wavefront partials of the weight gradients, (wave, enc, c, k): accumulator (enc, cq),
    // lane (blk, sub), component r is gW_enc[c = 4 cq + sub][k = 4 blk + r]
    if (NENC > 0) {
        float* dst = P.gw_partial + (size_t)blockIdx.x * 4 * DH * NBINS;
#pragma unroll
        for (int en = 0; en < NENC; en++) {
            const float sc = (en == 0 ? P.gw_dist_coef : P.angle_coef) * FIX_INV;
#pragma unroll
            for (int cq = 0; cq < 4; cq++) {
                const v4f_b acc = gWacc[en * 4 + cq];
                *reinterpret_cast<float4*>(dst + (en * DH + 4 * cq + sub) * NBINS + 4 * blk) =
                    make_float4(acc[0] * sc, acc[1] * sc, acc[2] * sc, acc[3] * sc);
            }
        }
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

// Rows of `bins` values <-> zero-padded rows of NBINS (the kernels are compiled for rows of NBINS bins; a basis of
// fewer bins runs on padded copies of its weights, and its weight gradients are taken back from padded rows).
// in/out: three tensors of `rows` rows each; thread per padded element.
__global__ __launch_bounds__(256) void pad_bins_kernel(const float* __restrict__ w1, const float* __restrict__ w2,
                                                       const float* __restrict__ w3, int rows, int bins,
                                                       float* __restrict__ padded) {
    const int idx = blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= 3 * rows * NBINS) return;
    const int k = idx % NBINS, r = (idx / NBINS) % rows, en = idx / (NBINS * rows);
    const float* w = en == 0 ? w1 : (en == 1 ? w2 : w3);
    padded[idx] = k < bins ? w[(size_t)r * bins + k] : 0.0f;
}
__global__ __launch_bounds__(256) void unpad_bins_kernel(const float* __restrict__ padded, int rows, int bins,
                                                         float* __restrict__ g1, float* __restrict__ g2,
                                                         float* __restrict__ g3) {
    const int idx = blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= 3 * rows * bins) return;
    const int k = idx % bins, r = (idx / bins) % rows, en = idx / (bins * rows);
    float* g = en == 0 ? g1 : (en == 1 ? g2 : g3);
    if (g) g[(size_t)r * bins + k] = padded[((size_t)en * rows + r) * NBINS + k];
}

}  // namespace cfh
