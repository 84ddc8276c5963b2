// Backward of the framed value position encoding when the forward pass kept its window histograms
// (KernelArgs::shat, 1 KB per (pair, head)): same mathematics and the same structure as
// framed_pe_bwd.hpp, but nothing is scattered -- the heavy pass only gathers sum_k g_k G_k for the
// gradient of a, and the weight gradients take the histogram bins from global memory.  Without the
// histograms in LDS a group holds 8 pairs (fuller lanes in the heavy pass) and the kernel issues no
// LDS atomics at all.  HBM pays for it: 4 x 64 floats per (pair, head) written by the forward and
// read here.
#pragma once
#include "framed_pe_bwd.hpp"

namespace cfh {

constexpr int GROUP_SAVED = 8;         // pairs per group: two rounds of four rows

// WITH_GW = false leaves the weight gradients to gw_from_histograms_kernel below (launched beside this
// kernel on a second stream): no accumulators, no histogram reads, no partials written here.
template <int WL, int WA, bool COS_ABS, bool HAS_LEN, bool HAS_ANG, bool WITH_GW = true>
__global__ __launch_bounds__(WAVE) void framed_pe_bwd_saved_kernel(const KernelArgs P) {
    __shared__ float4 tab[BWD_TCAP];
    __shared__ uint16_t list[BWD_LISTCAP];
    __shared__ __attribute__((aligned(16))) float Gs[GROUP_SAVED * PAIR_STRIDE];      // G per pair
    __shared__ __attribute__((aligned(16))) float gpS[GROUP_SAVED * DH];     // gpsi[p][c]
    __shared__ __attribute__((aligned(16))) float gpT[GROUP_SAVED * DH];     // gpsi[p][c] at (p*4 + c%4)*4 + c/4
    __shared__ float4 pairA[GROUP_SAVED];     // rx, ry, rz, A0
    __shared__ float pairZ[GROUP_SAVED];      // z * log2(e)

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
    v4f_b gWacc[(NENC > 0 && WITH_GW) ? NENC * 4 : 1];
#pragma unroll
    for (int en = 0; en < NENC; en++) {
#pragma unroll
        for (int c = 0; c < DH; c++) Wt[en * DH + c] = P.g_pair ? 0.0f : P.W[en][((size_t)h * DH + c) * NBINS + lane];
        if constexpr (WITH_GW) {
#pragma unroll
            for (int cq = 0; cq < 4; cq++) gWacc[en * 4 + cq] = v4f_b{0.f, 0.f, 0.f, 0.f};
        }
    }
    const BasisConsts bc = P.bc;
    const int WLr = WL > 0 ? WL : bc.len_window;      // bins of the distance window (WL == 0: known at run time only)
    const float prune = (P.prune_log2 > 0.0f) ? -P.prune_log2 : -3.0e38f;

    for (int u = lane; u < GROUP_SAVED * PAIR_STRIDE; u += WAVE) Gs[u] = 0.0f;
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
                    const int idx = lane * nb + bt;
                    if (idx < nlist) {
                        const uint32_t ent = list[idx];
                        const int el = ent >> BWD_SHIFT;
                        const float4 v = tab[ent & ((1u << BWD_SHIFT) - 1u)];
                        const float4 pa = pairA[el];
                        const float dx = pa.x + v.x, dy = pa.y + v.y, dz = pa.z + v.z;
                        const float d2 = fmaf(dx, dx, fmaf(dy, dy, dz * dz));
                        const float pf = hw_exp2(fmaf(a2, d2, -pairZ[el]));
                        const float* const myG = Gs + el * PAIR_STRIDE;
                        float pbg = 0.0f;
                        {
                            const float d = hw_sqrt(d2);
                            const float u = d * bc.inv_interval;
                            int start = (int)(u - bc.start_off);
                            start = max(0, min(start, NBINS - WLr));
                            const float beta_c = ((float)(start + WLr / 2 + 1) - u) * bc.len_step;
                            const WindowSeed s = window_seed(beta_c, bc.len_step, pf);
                            pbg += window_gather<WL>(myG + start, s, bc.len_cc, WLr);
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
                                    pbg += window_gather<WA>(myG + (ax + 1) * HS + start, s, bc.ang_cc);
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

        // ---- weight gradients of the ng pairs of the finished group, histograms from the forward pass
        auto gw_update = [&](int g0, int ng) {
            if constexpr (NENC > 0 && WITH_GW) {
                for (int p = 0; p < ng; p++) {
                    const float4 gq = reinterpret_cast<const float4*>(gpT)[p * 4 + sub];   // gpsi[p][4 cq + sub]
                    const float* sp = P.shat + (((size_t)(g0 + p) * H + h) * 4) * NBINS + lane;
                    float sk[NENC > 0 ? NENC : 1];
                    // read once: streaming loads, so that the L2 keeps what is used again
#pragma unroll
                    for (int en = 0; en < NENC; en++) sk[en] = __builtin_nontemporal_load(sp + en * NBINS);
#pragma unroll
                    for (int en = 0; en < NENC; en++) {
                        gWacc[en * 4 + 0] = __builtin_amdgcn_mfma_f32_4x4x1f32(sk[en], gq.x, gWacc[en * 4 + 0], 0, 0, 0);
                        gWacc[en * 4 + 1] = __builtin_amdgcn_mfma_f32_4x4x1f32(sk[en], gq.y, gWacc[en * 4 + 1], 0, 0, 0);
                        gWacc[en * 4 + 2] = __builtin_amdgcn_mfma_f32_4x4x1f32(sk[en], gq.z, gWacc[en * 4 + 2], 0, 0, 0);
                        gWacc[en * 4 + 3] = __builtin_amdgcn_mfma_f32_4x4x1f32(sk[en], gq.w, gWacc[en * 4 + 3], 0, 0, 0);
                    }
                }
            }
            wave_sync();               // gpS/gpT and pair data are free again
        };

        // ---- rounds: 4 pairs of the group of 8 (one per row), chunk ch of the translations
        float prx = 0.f, pry = 0.f, prz = 0.f, pz2 = 0.f, pgz = 0.f;   // pair (row base + lane)
        float4 pgp = make_float4(0.f, 0.f, 0.f, 0.f);                  // gpsi of pair (block base + lane/4), channels 4 (lane%4)..
        float rx = 0.f, ry = 0.f, rz = 0.f, z2 = 0.f, gzr = 0.f, A0 = 0.f;
        int cur_g0 = -1, cur_ng = 0;
        int el_glob = 0, ch = 0;
        int skip = 0;          // survivors of the current round already processed (list overflow)
        while (true) {
            const bool done = el_glob >= npairs;
            const int g0n = done ? -2 : e0 + (el_glob / GROUP_SAVED) * GROUP_SAVED;
            const bool group_change = g0n != cur_g0;
            if (nlist > 0 && (group_change || nchunks > 1 || skip > 0)) flush();
            if (group_change && cur_g0 >= 0) gw_update(cur_g0, cur_ng);
            if (done) break;
            const int el = (el_glob & (GROUP_SAVED - 1)) + slot;   // pair-in-group of this row of lanes
            if (group_change) {
                cur_g0 = g0n;
                cur_ng = min(GROUP_SAVED, e1 - g0n);
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
                        if (e < e1 && !P.g_pair)
                            pgp = reinterpret_cast<const float4*>(P.gpsi + ((size_t)e * H + h) * DH)[sub];
                    }
                    // the 32 lanes that hold this group's gpsi stage it in both layouts
                    if (((lane >> 5) << 3) == (el_glob & 15)) {
                        const int p = (lane >> 2) & 7;
                        reinterpret_cast<float4*>(gpS)[p * 4 + sub] = pgp;
                        gpT[(p * 4 + 0) * 4 + sub] = pgp.x;
                        gpT[(p * 4 + 1) * 4 + sub] = pgp.y;
                        gpT[(p * 4 + 2) * 4 + sub] = pgp.z;
                        gpT[(p * 4 + 3) * 4 + sub] = pgp.w;
                    }
                    wave_sync();
                    // G[pair = 4 half + sub][enc][k = 4 blk + r] = sum_c W_enc[c][k] gpsi[pair][c]
                    if (P.g_pair) {          // given per pair (already scaled by the encodings' coefficients)
                        for (int half = 0; half * 4 < cur_ng; half++) {
                            const int pl = half * 4 + sub;
                            const float4* src = reinterpret_cast<const float4*>(
                                P.g_pair + (((size_t)(cur_g0 + min(pl, cur_ng - 1)) * H + h) * 4) * NBINS) + blk;
#pragma unroll
                            for (int en = 0; en < NENC; en++)
                                *reinterpret_cast<float4*>(Gs + pl * PAIR_STRIDE + en * HS + 4 * blk) = src[en * (NBINS / 4)];
                        }
                    } else
                    for (int half = 0; half * 4 < cur_ng; half++) {
                        const int pl = half * 4 + sub;
                        float gb[DH];
#pragma unroll
                        for (int c4 = 0; c4 < DH / 4; c4++) {
                            const float4 t4 = reinterpret_cast<const float4*>(gpS)[pl * 4 + c4];
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
                            const float sc = (en == 0 ? P.dist_coef : P.angle_coef);
                            *reinterpret_cast<float4*>(Gs + pl * PAIR_STRIDE + en * HS + 4 * blk) =
                                make_float4(g[en][0] * sc, g[en][1] * sc, g[en][2] * sc, g[en][3] * sc);
                        }
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
                    uint32_t bits = 0u;
#pragma unroll
                    for (int k = 0; k < 8; k++) {
                        const bool valid = active && tl + 16 * k < cnt;
                        const float ex = fmaf(a2, d2r[k], -z2);
                        Ap += valid ? hw_exp2(ex) * d2r[k] : 0.0f;
                        bits |= (valid && ex >= prune) ? (1u << k) : 0u;
                    }
                    seen = append_flagged(list, nlist, room, skip, bits, slot, (uint32_t)((el << BWD_SHIFT) | tl));
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
                el_glob += 4;
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
    if constexpr (NENC > 0 && WITH_GW) {
        float* dst = P.gw_partial + (size_t)blockIdx.x * 4 * DH * NBINS;
#pragma unroll
        for (int en = 0; en < NENC; en++) {
            const float sc = (en == 0 ? P.gw_dist_coef : P.angle_coef);
#pragma unroll
            for (int cq = 0; cq < 4; cq++) {
                const v4f_b acc = gWacc[en * 4 + cq];
                *reinterpret_cast<float4*>(dst + (en * DH + 4 * cq + sub) * NBINS + 4 * blk) =
                    make_float4(acc[0] * sc, acc[1] * sc, acc[2] * sc, acc[3] * sc);
            }
        }
    }
}

// The weight gradients from the kept histograms alone,
//     gW_enc[h, c, k] = sum over the pairs e of gpsi[e, h, c] shat[e, h, enc, k],
// a stream of 1 KB + 64 B per (pair, head) with nothing else to compute: launched on a second stream beside
// framed_pe_bwd_saved_kernel<..., false>, whose wavefronts leave a quarter of the registers of every SIMD
// free, it overlaps its memory traffic with their arithmetic.  Workgroup w (one wavefront) serves head
// w % H and the pairs of slice w / H; lane = bin for the histogram operand, 4 pairs in flight; partials
// in the layout gw_reduce_kernel sums.  grid: H * nslices.
constexpr int GWH_UNROLL = 4;
template <bool HAS_ANG>
__global__ __launch_bounds__(WAVE) void gw_from_histograms_kernel(const float* __restrict__ shat,
                                                                  const float* __restrict__ gpsi, int E, int H,
                                                                  int nslices, float dist_scale, float angle_scale,
                                                                  float* __restrict__ partial) {
    constexpr int NENC = HAS_ANG ? 4 : 1;
    const int lane = threadIdx.x;
    const int sub = lane & 3, blk = lane >> 2;
    const int h = blockIdx.x % H, slice = blockIdx.x / H;
    const int per = (E + nslices - 1) / nslices;
    const int e0 = min(E, slice * per), e1 = min(E, e0 + per);
    v4f_b acc[NENC * 4];
#pragma unroll
    for (int u = 0; u < NENC * 4; u++) acc[u] = v4f_b{0.f, 0.f, 0.f, 0.f};
    for (int e = e0; e < e1; e += GWH_UNROLL) {
        float sk[GWH_UNROLL][NENC];
        float gq[GWH_UNROLL][4];
#pragma unroll
        for (int u = 0; u < GWH_UNROLL; u++) {
            const bool live = e + u < e1;
            const size_t row = (size_t)(live ? e + u : e) * H + h;
            const float* sp = shat + row * 4 * NBINS + lane;
            const float* gp = gpsi + row * DH + sub;
#pragma unroll
            for (int en = 0; en < NENC; en++) sk[u][en] = live ? __builtin_nontemporal_load(sp + en * NBINS) : 0.0f;
#pragma unroll
            for (int cq = 0; cq < 4; cq++) gq[u][cq] = live ? gp[4 * cq] : 0.0f;      // gpsi[e][4 cq + sub]
        }
#pragma unroll
        for (int u = 0; u < GWH_UNROLL; u++)
#pragma unroll
            for (int en = 0; en < NENC; en++)
#pragma unroll
                for (int cq = 0; cq < 4; cq++)
                    acc[en * 4 + cq] = __builtin_amdgcn_mfma_f32_4x4x1f32(sk[u][en], gq[u][cq], acc[en * 4 + cq], 0, 0, 0);
    }
    // accumulator (enc, cq), lane (blk, sub), component r is gW_enc[c = 4 cq + sub][k = 4 blk + r]
    float* dst = partial + (size_t)blockIdx.x * 4 * DH * NBINS;
#pragma unroll
    for (int en = 0; en < NENC; en++) {
        const float sc = en == 0 ? dist_scale : angle_scale;
#pragma unroll
        for (int cq = 0; cq < 4; cq++) {
            const v4f_b a = acc[en * 4 + cq];
            *reinterpret_cast<float4*>(dst + (en * DH + 4 * cq + sub) * NBINS + 4 * blk) =
                make_float4(a[0] * sc, a[1] * sc, a[2] * sc, a[3] * sc);
        }
    }
}

}  // namespace cfh
