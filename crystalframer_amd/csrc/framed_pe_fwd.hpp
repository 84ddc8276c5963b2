// Forward of the framed value position encoding: z, psi (and optionally d2min) for every
// (pair, head).  One launch covers what the reference does in two kernels plus a tensor sum
// (models/kernels/real_enc_frame_proj_fwd_length.cu, ..._fwd_angle.cu,
//  models/cuda_funcs/real_space_framed_proj.py:63-105).
//
// Per (atom i, head h) item, pairs e=(i,j) taken GROUP at a time:
//   rounds of up to 4 pairs, one pair per 16-lane row, lanes of a row over the translations n:
//     pass A  d2min = min_n |r_ij + n.L|^2                     (row reduction in DPP, no LDS)
//     pass B  w_n = 2^(a'(d^2-d2min)); S = sum_n w_n; the translations with w_n >= 2^-prune are
//             appended (ballot/prefix compaction) to the group's LDS list
//   per group, lanes over the list:
//     pass C  p = w/S; scatter p*g_k(d) into the pair's 9-bin distance window and p*g_m(cos(n,f_axis))
//             into its three 33-bin angle windows (fixed-point LDS adds, Gaussians by recurrence)
//   per 4 pairs of the group:
//     epilogue psi[pair, c] = sum_enc sum_k W_enc[h,c,k] hist[pair,enc,k] as 64 MFMA 4x4x1 steps:
//             block (enc, c/4) of the instruction multiplies the 4 channels of its lanes' weight
//             rows (held in registers for the whole launch) with the bins of 4 pairs;
//             z = log S + a d2min.
#pragma once
#include "device_common.hpp"

namespace cfh {

constexpr int FWD_TCAP = 256;          // translations staged in LDS at a time (4 KB)
constexpr int FWD_LISTCAP = 512;       // entries of the survivor list (a round that overflows it is repeated)
constexpr int FWD_SHIFT = 13;          // list entry = pair-in-group << 13 | table index
constexpr int FWD_ROWS = 4;            // pairs per round, one per 16-lane row
constexpr int FAST_PER_LANE = 8;       // boxes of up to 128 translations: 8 per lane of a row, kept in registers
static_assert(FWD_TCAP <= (1 << FWD_SHIFT) && (GROUP << FWD_SHIFT) <= 65536, "list entry is 16 bits");
static_assert(GROUP % FWD_ROWS == 0 && WAVE % GROUP == 0, "rounds must not straddle groups or 64-pair rows");

typedef float v4f __attribute__((ext_vector_type(4)));

template <int WL, int WA, bool COS_ABS, bool HAS_LEN, bool HAS_ANG>
__global__ __launch_bounds__(WAVE) void framed_pe_fwd_kernel(const KernelArgs P) {
    __shared__ float4 tab[FWD_TCAP];
    __shared__ uint16_t list[FWD_LISTCAP];
    __shared__ __attribute__((aligned(16))) uint32_t hist[GROUP * PAIR_STRIDE];
    __shared__ float4 pairA[GROUP];        // rx, ry, rz, d2min of the pairs of the group
    __shared__ float2 pairS[GROUP];        // S and 2^31/S

    const int lane = threadIdx.x;
    const int H = P.H;
    const int h = blockIdx.x % H;
    const int enc = lane >> 4;        // epilogue: 0 = distance, 1..3 = frame axes
    const int c = lane & 15;          // epilogue: output channel of this lane's weight row
    const int slot = lane >> 4;       // passes A/B: which pair of the round
    const int tl = lane & 15;         // passes A/B: position in the row

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
    const float enc_scale = ((enc == 0) ? P.dist_coef : P.angle_coef) * FIX_INV;
    const BasisConsts bc = P.bc;
    const int WLr = WL > 0 ? WL : bc.len_window;      // bins of the distance window (WL == 0: known at run time only)
    const float prune = (P.prune_log2 > 0.0f) ? -P.prune_log2 : -3.0e38f;

    for (int u = lane; u < GROUP * PAIR_STRIDE; u += WAVE) hist[u] = 0u;
    wave_sync();

    unsigned long long st_eval = 0, st_raw = 0, st_pairs = 0;
    // software pipeline over items: while item n is processed, the record of item n+1 and the
    // queue ticket of item n+2 are in flight
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
        const int nchunks = (bx.T + FWD_TCAP - 1) / FWD_TCAP;
        // boxes of up to 128 translations with a < 0: one slab of 8 per lane, distances stay in
        // registers between the passes; the table is padded with infinitely distant shifts, whose weight
        // 2^(a d^2) is exactly zero, so that the slab needs no bounds checks
        const bool fast = bx.T <= 16 * FAST_PER_LANE && a2 < 0.0f;
        if (nchunks == 1) {
            wave_sync();
            build_shift_table(tab, 0, bx.T, bx, L, lane);
            if (fast)
                for (int u = bx.T + lane; u < 16 * FAST_PER_LANE; u += WAVE)
                    tab[u] = make_float4(__builtin_inff(), 0.0f, 0.0f, 0.0f);
            wave_sync();
        }
        const int e0 = item.e0;
        const int npairs = item.npairs;
        const int e1 = e0 + npairs;
        unsigned long long n_eval = 0;
        int nlist = 0;

        // ---- pass C over the current list; the table the entries point into is still resident
        auto flush = [&]() {
            wave_sync();                           // list and pair data written
            if (HAS_LEN) {
                const int nb = (nlist + WAVE - 1) / WAVE;
                for (int bt = 0; bt < nb; bt++) {
                    // every nb-th entry, and neighbouring entries (mostly translations of one pair, which
                    // often share a clamped window and then add to the same words) in different 16-lane rows
                    const int idx = (((lane & 15) << 2) | (lane >> 4)) * nb + bt;
                    if (idx < nlist) {
                        const uint32_t ent = list[idx];
                        const int el = ent >> FWD_SHIFT;
                        const float4 v = tab[ent & ((1u << FWD_SHIFT) - 1u)];
                        const float4 pa = pairA[el];
                        const float dx = pa.x + v.x, dy = pa.y + v.y, dz = pa.z + v.z;
                        const float d2 = fmaf(dx, dx, fmaf(dy, dy, dz * dz));
                        const float w = hw_exp2(a2 * (d2 - pa.w)) * pairS[el].y;
                        uint32_t* const myhist = hist + el * PAIR_STRIDE;
                        const int dir = ((lane ^ (lane >> 4)) & 1) ? -1 : 1;     // half of the lanes walk their windows the other way round
                        {
                            const float d = hw_sqrt(d2);
                            const float u = d * bc.inv_interval;
                            int start = (int)(u - bc.start_off);          // truncation toward zero
                            start = max(0, min(start, NBINS - WLr));
                            // bin k has centre (k+1)*interval: scaled offset ((k+1) - u)*len_step
                            const float beta_c = ((float)(start + WLr / 2 + 1) - u) * bc.len_step;
                            const WindowSeed s = window_seed(beta_c, bc.len_step, w);
                            window_scatter_dir<WL>(myhist + start, s, bc.len_cc, dir, WLr);
                        }
                        if (HAS_ANG) {
                            if (d2 > 1e-5f) {       // the self image contributes to S only
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
                                    const WindowSeed s = window_seed(beta_c, bc.ang_step, w);
                                    window_scatter_dir<WA>(myhist + (ax + 1) * HS + start, s, bc.ang_cc, dir);
                                }
                            }
                        }
                    }
                }
            }
            n_eval += (unsigned long long)nlist;
            nlist = 0;
            wave_sync();                           // list may be refilled, histograms may be read
        };

        // ---- projection of the histograms of group g0 (ng pairs), stores, histograms cleared
        auto epilogue = [&](int g0, int ng) {
            if (HAS_LEN) {
                const int sub = lane & 3;          // A row of this lane: a pair; B column: channel 4 cg + sub
                const int cg = (lane >> 2) & 3;
                for (int half = 0; half * 4 < ng; half++) {
                    // block (enc, cg) supplies the bins 16 cg .. 16 cg + 15 of its encoding; each of the
                    // four MFMA of a step broadcasts the A operand of one cg to all four blocks of enc
                    uint4* hb = reinterpret_cast<uint4*>(hist + (half * 4 + sub) * PAIR_STRIDE + enc * HS + 16 * cg);
                    float hv[16];
#pragma unroll
                    for (int k4 = 0; k4 < 4; k4++) {
                        const uint4 t4 = hb[k4];
                        hb[k4] = make_uint4(0u, 0u, 0u, 0u);
                        hv[4 * k4 + 0] = (float)t4.x; hv[4 * k4 + 1] = (float)t4.y;
                        hv[4 * k4 + 2] = (float)t4.z; hv[4 * k4 + 3] = (float)t4.w;
                    }
                    if (P.shat && half * 4 + sub < ng) {
                        // keep the histograms for the backward pass: this lane's 16 bins of (pair, enc)
                        float4* dst = reinterpret_cast<float4*>(
                            P.shat + (((size_t)(g0 + half * 4 + sub) * H + h) * 4 + enc) * NBINS + 16 * cg);
#pragma unroll
                        for (int k4 = 0; k4 < 4; k4++)
                            dst[k4] = make_float4(hv[4 * k4 + 0] * FIX_INV, hv[4 * k4 + 1] * FIX_INV,
                                                  hv[4 * k4 + 2] * FIX_INV, hv[4 * k4 + 3] * FIX_INV);
                    }
                    v4f acc0 = {0.f, 0.f, 0.f, 0.f}, acc1 = {0.f, 0.f, 0.f, 0.f};
                    v4f acc2 = {0.f, 0.f, 0.f, 0.f}, acc3 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                    for (int s = 0; s < 16; s++) {
                        acc0 = __builtin_amdgcn_mfma_f32_4x4x1f32(hv[s], Wrow[s], acc0, 2, 0, 0);
                        acc1 = __builtin_amdgcn_mfma_f32_4x4x1f32(hv[s], Wrow[16 + s], acc1, 2, 1, 0);
                        acc2 = __builtin_amdgcn_mfma_f32_4x4x1f32(hv[s], Wrow[32 + s], acc2, 2, 2, 0);
                        acc3 = __builtin_amdgcn_mfma_f32_4x4x1f32(hv[s], Wrow[48 + s], acc3, 2, 3, 0);
                    }
                    // lane (enc, c = lane & 15), component r: pair half*4 + r
#pragma unroll
                    for (int r = 0; r < 4; r++) {
                        const float x = rows_sum(((acc0[r] + acc1[r]) + (acc2[r] + acc3[r])) * enc_scale);
                        if (lane < DH && half * 4 + r < ng)
                            P.out_psi[((size_t)(g0 + half * 4 + r) * H + h) * DH + lane] = x;
                    }
                }
            }
            if (lane < ng) {
                const float4 pa = pairA[lane];
                P.out_z[(size_t)(g0 + lane) * H + h] = logf(pairS[lane].x) + pa.w * a;
                if (P.out_d2min) P.out_d2min[(size_t)(g0 + lane) * H + h] = pa.w;
            }
            wave_sync();                           // pair data of this group no longer needed
        };

        // ---- rounds: (pairs el_glob .. el_glob+nslots of the row, chunk ch of the translations)
        float prx = 0.f, pry = 0.f, prz = 0.f;     // rpos of pair (row base + lane)
        float rx = 0.f, ry = 0.f, rz = 0.f, d2min = 0.f, S = 0.f;
        int cur_g0 = -1, cur_ng = 0;
        int el_glob = 0, ch = 0;
        int skip = 0;          // survivors of the current round already processed (list overflow)
        float d2r[FAST_PER_LANE];
#pragma unroll
        for (int k = 0; k < FAST_PER_LANE; k++) d2r[k] = 0.0f;
        while (true) {
            const bool done = el_glob >= npairs;
            const int g0n = done ? -2 : e0 + (el_glob / GROUP) * GROUP;
            const bool group_change = g0n != cur_g0;
            if (nlist > 0 && (group_change || nchunks > 1 || skip > 0)) flush();
            if (group_change && cur_g0 >= 0) epilogue(cur_g0, cur_ng);
            if (done) break;
            if (group_change) { cur_g0 = g0n; cur_ng = min(GROUP, e1 - g0n); }
            if ((el_glob & (WAVE - 1)) == 0 && ch == 0) {      // next 64 pairs of the row
                const int e = e0 + el_glob + lane;
                if (e < e1) {
                    prx = P.rpos[(size_t)e * 3 + 0];
                    pry = P.rpos[(size_t)e * 3 + 1];
                    prz = P.rpos[(size_t)e * 3 + 2];
                }
            }
            const int el = (el_glob & (GROUP - 1)) + slot;      // pair-in-group of this row of lanes
            const bool active = el < cur_ng;

            if (ch == 0) {
                const int src = (el_glob & (WAVE - 1)) + min(slot, WAVE - 1 - (el_glob & (WAVE - 1)));
                rx = __shfl(prx, src, WAVE);
                ry = __shfl(pry, src, WAVE);
                rz = __shfl(prz, src, WAVE);
                // ---- pass A: nearest image
                d2min = 3.0e38f;
                if (fast) {
                    // every lane keeps the squared distances of its 8 translations for pass B
#pragma unroll
                    for (int k = 0; k < FAST_PER_LANE; k++) {
                        const float4 v = tab[tl + 16 * k];
                        const float dx = rx + v.x, dy = ry + v.y, dz = rz + v.z;
                        d2r[k] = fmaf(dx, dx, fmaf(dy, dy, dz * dz));
                        d2min = fminf(d2min, d2r[k]);
                    }
                } else {
                    for (int cc = 0; cc < nchunks; cc++) {
                        const int t0 = cc * FWD_TCAP;
                        const int cnt = min(FWD_TCAP, bx.T - t0);
                        if (nchunks > 1) {
                            wave_sync();
                            build_shift_table(tab, t0, cnt, bx, L, lane);
                            wave_sync();
                        }
                        for (int u = tl; u < cnt; u += 16) {
                            const float4 v = tab[u];
                            const float dx = rx + v.x, dy = ry + v.y, dz = rz + v.z;
                            d2min = fminf(d2min, fmaf(dx, dx, fmaf(dy, dy, dz * dz)));
                        }
                    }
                }
                d2min = row_min(d2min);
                // ---- the normaliser S when the table does not fit at once (otherwise pass B gives it)
                if (nchunks > 1) {
                    float Sb = 0.0f;
                    for (int cc = 0; cc < nchunks; cc++) {
                        const int t0 = cc * FWD_TCAP;
                        const int cnt = min(FWD_TCAP, bx.T - t0);
                        wave_sync();
                        build_shift_table(tab, t0, cnt, bx, L, lane);
                        wave_sync();
                        for (int u = tl; u < cnt; u += 16) {
                            const float4 v = tab[u];
                            const float dx = rx + v.x, dy = ry + v.y, dz = rz + v.z;
                            Sb += hw_exp2(a2 * (fmaf(dx, dx, fmaf(dy, dy, dz * dz)) - d2min));
                        }
                    }
                    S = row_sum(Sb);
                    if (active && tl == 0) {
                        pairA[el] = make_float4(rx, ry, rz, d2min);
                        pairS[el] = make_float2(S, FIX_ONE / S);
                    }
                }
            }

            // ---- pass B on chunk ch: weights, normaliser, compaction of the translations that matter
            {
                const int t0 = ch * FWD_TCAP;
                const int cnt = min(FWD_TCAP, bx.T - t0);
                if (nchunks > 1) {
                    wave_sync();
                    build_shift_table(tab, t0, cnt, bx, L, lane);
                    wave_sync();
                }
                float Sb = 0.0f;
                const int room = FWD_LISTCAP - nlist;
                int seen = 0;                      // survivors met so far in this round
                if (fast) {
                    uint32_t bits = 0u;
#pragma unroll
                    for (int k = 0; k < FAST_PER_LANE; k++) {
                        const float ex = a2 * (d2r[k] - d2min);          // -inf for the padding
                        Sb += hw_exp2(ex);
                        bits |= (ex >= prune) ? (1u << k) : 0u;
                    }
                    if (!active) bits = 0u;
                    seen = append_flagged(list, nlist, room, skip, bits, slot, (uint32_t)((el << FWD_SHIFT) | tl));
                } else {
                    for (int u0 = 0; u0 < cnt; u0 += 16) {
                        const int u = u0 + tl;
                        bool keep = false;
                        if (active && u < cnt) {
                            const float4 v = tab[u];
                            const float dx = rx + v.x, dy = ry + v.y, dz = rz + v.z;
                            const float ex = a2 * (fmaf(dx, dx, fmaf(dy, dy, dz * dz)) - d2min);
                            Sb += hw_exp2(ex);
                            keep = ex >= prune;
                        }
                        const uint64_t m = __ballot(keep);
                        const int pos = seen + lane_prefix(m) - skip;
                        if (keep && pos >= 0 && pos < room) list[nlist + pos] = (uint16_t)((el << FWD_SHIFT) | u);
                        seen += __popcll(m);
                    }
                }
                const int appended = min(seen - skip, room);
                nlist += appended;
                skip = (skip + appended < seen) ? skip + appended : 0;   // > 0: repeat the round after a flush
                if (nchunks == 1) {
                    S = row_sum(Sb);
                    if (active && tl == 0) {
                        pairA[el] = make_float4(rx, ry, rz, d2min);
                        pairS[el] = make_float2(S, FIX_ONE / S);
                    }
                }
            }
            if (skip == 0 && ++ch == nchunks) { ch = 0; el_glob += FWD_ROWS; }
        }
        st_eval += n_eval;
        st_raw += (unsigned long long)bx.T * (unsigned long long)npairs;
        st_pairs += (unsigned long long)npairs;
        (void)i;
        it_cur = it_next;
        rec_cur = rec_next;
        it_next = it_cur >= 0 ? queue_redeem(P, h, queue, ticket) : -1;
    }
    // one set of atomics per wavefront (per-item atomics on three shared addresses serialise in L2)
    if (P.stats && lane == 0) {
        atomicAdd(P.stats + STAT_FWD_EVAL, st_eval);
        atomicAdd(P.stats + STAT_FWD_RAW, st_raw);
        atomicAdd(P.stats + STAT_FWD_PAIRS, st_pairs);
    }
}

}  // namespace cfh
