// "Max" frame selection over translations sorted by length (both axes, Gram-Schmidt and cross product in one
// launch).  Same arg-maxima, tie rule and noise as frame_axis_kernel<2> (frame_select.hpp; reference:
// models/kernels/compute_maximum_frame_each_edge.cu:78-111, compute_second_frame_each_edge.cu:81-142,
// models/cuda_funcs/calc_maximum_frame.py:72-86,146-164), found by looking at far fewer candidates.
//
// With the shifts of a crystal's box sorted by length |s| (one table per crystal, sorted_shifts_kernel), an image
// of pair (i,j) at shift s lies at distance d with  |s| - |r_ij| <= d <= |s| + |r_ij|.  For a < 0:
//   * first axis: the best candidate of a pair is its nearest valid image (d^2 > 1e-5).  The unshifted image is at
//     distance |r|, so the nearest one has |s| <= 2 |r|; when the unshifted image is the atom itself (|r| = 0) the
//     shortest non-zero shift s_1 gives d <= |r| + |s_1|, hence |s| <= 2 |r| + |s_1|.  Only that prefix is read.
//     With the batch's table of every pair's nearest valid image (pair_nearest_kernel: its d^2 and its position in
//     the sorted table) most pairs are not looked at at all: no candidate of pair j scores above
//     hi_j = q.k_j + a (d_j^2 - noise / 2), and its nearest valid image scores at least lo_j = q.k_j + a (d_j^2 + noise / 2),
//     so only the pairs with hi_j >= max_j lo_j can hold the maximum -- one or two of a row, unless images tie.
//   * second axis: score = q.k + a d^2 + log(max(1 - |cos|, 1e-5)) <= q.k + a d^2.  A first sweep -- over every
//     pair's nearest valid image when the batch's table names it, else over the first axis' prefixes -- gives a
//     lower bound `best` of the maximum; a candidate of pair j can then only matter if
//     a d^2 >= best - q.k_j, i.e. d^2 <= need_j = (best - q.k_j) / a: no candidate when need_j < 0, else only
//     shifts with |s| <= |r| + sqrt(need_j).  The second sweep reads those prefixes.
// The tie-breaking noise moves a score by at most |a| noise / 2 (first axis) or noise / 2 (second): the bounds are
// widened by that much.  Items whose box is not the table's (or a >= 0) scan their whole box, a chunk at a time.
//
// Layout: the candidates of up to 64 pairs are laid end to end -- pair j contributes the first cnt_j entries of the
// sorted table, cnt_j found by bisection of the lengths -- and dealt to the lanes 64 at a time, so the lanes stay
// full whatever the prefixes are (a lane finds its pair by bisection of the prefix sums).  Every lane keeps its best
// (score, pair, translation); one wavefront reduction per axis.
#pragma once
#include "frame_select.hpp"
#include "fused_core.hpp"

namespace cfh {

constexpr int FQ_ROWS = 4;          // heads of an atom per wavefront, one per 16-lane row
constexpr int FQ_STAGE = 16;        // pairs staged at a time (the rows of this search have no more)
constexpr int FQ_PAIR_GROUP = 16;   // pairs of a row whose candidates are laid end to end at a time (one per lane of the row)
constexpr int FQ_MAX_PAIRS = 16;    // longer rows go one item per wavefront: 64 lanes finish a long item sooner than 16
static_assert(FQ_MAX_PAIRS <= FQ_STAGE && FQ_STAGE <= WAVE, "a row of the four-heads search is staged as a whole");

// Shifts t0 .. t0+cnt (cnt <= 128) of the box, sorted by length within the chunk: w = length with the position in the
// chunk (loop order of the reference) in its low 7 bits, like the entries of the per-crystal tables.  Items whose box
// is not the table's thereby get the same bounded prefixes, chunk by chunk (a bound on the distance of a candidate
// holds for any subset of the translations).  Each lane makes two entries and ranks them against all keys.
__device__ __forceinline__ void build_sorted_chunk(float4* tab, int t0, int cnt, const Box& bx, const Lattice& L, int lane) {
    float4 ent[2];
#pragma unroll
    for (int k = 0; k < 2; k++) {
        const int u = lane + k * WAVE;
        const int t = t0 + min(u, cnt - 1);
        const int i3 = t % bx.s3;
        const int q = t / bx.s3;
        const int i2 = q % bx.s2;
        const int i1 = q / bx.s2;
        const float n1 = (float)(i1 - bx.R1), n2 = (float)(i2 - bx.R2), n3 = (float)(i3 - bx.R3);
        float4 v;
        v.x = fmaf(L.t[6], n3, fmaf(L.t[3], n2, L.t[0] * n1));
        v.y = fmaf(L.t[7], n3, fmaf(L.t[4], n2, L.t[1] * n1));
        v.z = fmaf(L.t[8], n3, fmaf(L.t[5], n2, L.t[2] * n1));
        const float len = sqrtf(fmaf(v.x, v.x, fmaf(v.y, v.y, v.z * v.z)));
        v.w = u < cnt ? __uint_as_float((__float_as_uint(len) & ~(uint32_t)(FC_TCAP - 1)) | (uint32_t)u) : __builtin_inff();
        ent[k] = v;
        tab[u] = v;
    }
    wave_sync();
    int rank[2] = {0, 0};
    // (entries beyond cnt hold +inf and count for nobody; eight reads in flight: the loop waited for one LDS round
    // trip per key otherwise)
#pragma unroll 8
    for (int j = 0; j < FC_TCAP; j++) {
        const float kj = tab[j].w;         // the keys differ in their low bits: no ties
        rank[0] += kj < ent[0].w ? 1 : 0;
        rank[1] += kj < ent[1].w ? 1 : 0;
    }
    wave_sync();
    if (lane < cnt) tab[rank[0]] = ent[0];
    if (lane + WAVE < cnt) tab[rank[1]] = ent[1];
    for (int u = cnt + lane; u < FC_TCAP; u += WAVE) tab[u] = make_float4(0.f, 0.f, 0.f, __builtin_inff());
}

struct FrameShared {
    float4 tab[2 * FC_TCAP];     // the sorted table, or the sorted chunks of a box of its own (two stay resident)
    float4 pq[WAVE];             // rpos and q.k of the staged pairs
    uint32_t markw[WAVE * FC_TCAP / 32];      // one bit per candidate, set where the run of a pair begins
    uint32_t ent[WAVE];          // the staged pairs that have candidates, in order: first candidate | pair << 16
    float ph[WAVE];              // phase of the tie-breaking noise of the staged pairs in the current pass
    int total;                   // candidates of the list that the marks describe
};
// one wavefront, one item: wid = item * H + head.  `others_only`: only the items that the four-heads-per-wavefront
// search leaves out (box not the table's, or more pairs than it takes).
// `skip_listed`: the records listed for the first wavefronts of the launch are theirs.
__device__ __forceinline__ void frame_item_body(const CoreArgs& C, FrameShared& sh, int wid, int lane, bool others_only,
                                                bool skip_listed) {
    float4* const tab = sh.tab;
    float4* const pq = sh.pq;
    uint32_t* const markw = sh.markw;
    uint32_t* const ent = sh.ent;

    const KernelArgs& P = C.K;
    const int H = P.H;
    const int it_cur = div_heads(P, wid);      // one wavefront per item, long items first
    const int h = wid - it_cur * H;
    const bool noisy = P.noise > 0.0f;
    uint32_t seed_lo = P.seed_lo, seed_hi = P.seed_hi;
    if (noisy && P.seed_dev) {
        const unsigned long long s = *P.seed_snap;
        seed_lo ^= (uint32_t)s * 0x9E3779B1u;
        seed_hi += (uint32_t)(s >> 32) ^ ((uint32_t)s * 0x85EBCA77u);
    }

    if (it_cur >= P.N) return;
    {
        const uint32_t rec_cur = load_record_lane(P, it_cur, h, lane);
        if (skip_listed && ((uint32_t)__builtin_amdgcn_readlane((int)rec_cur, REC_BOX) & REC_BOX_LISTED) != 0u &&
            core_slow_rank(C, wid, lane) < C.slow_wgs)
            return;      // (a listed record of higher rank stays here)
        const Item item = unpack_item(rec_cur);
        const int crystal = __builtin_amdgcn_readlane((int)rec_cur, REC_CRYSTAL);
        const int j0 = __builtin_amdgcn_readlane((int)rec_cur, REC_J0);
        const int i = item.i;
        const float a = item.a;
        const float inv_a = a < 0.0f ? hw_rcp(a) : 0.0f;      // (for a reach with margins: the hardware reciprocal will do)
        const Lattice L = item.L;
        const Box bx = item.bx;
        float qi[DH];
#pragma unroll
        for (int c = 0; c < DH; c++) qi[c] = rec_f(rec_cur, REC_QUERY + c);
        const bool sorted = C.sorted_tab != nullptr && bx.R1 == C.table_R && bx.R2 == C.table_R && bx.R3 == C.table_R &&
                            a < 0.0f;
        if (others_only && sorted && item.npairs <= FQ_MAX_PAIRS) return;      // searched four heads at a time
        const int nchunks = sorted ? 1 : (bx.T + FC_TCAP - 1) / FC_TCAP;
        const bool resident = nchunks == 2;             // both chunks of the box fit: sorted once, not once per sweep
        const int e0 = item.e0, npairs = item.npairs;
        const float nz = noisy ? P.noise : 0.0f;
        const float sq_nz = sqrtf(nz);

        if (sorted) {
            const float4* src = C.sorted_tab + (size_t)crystal * FC_TCAP;
            tab[lane] = src[lane];
            tab[lane + WAVE] = src[lane + WAVE];
        } else if (nchunks == 1) {
            build_sorted_chunk(tab, 0, bx.T, bx, L, lane);
        }
        wave_sync();
        const float s1 = sorted ? tab[1].w : 0.0f;      // shortest non-zero shift (entry 0 is the zero shift)

        float dvalid = -1.0f;                           // this lane's pair: d^2 of its nearest valid image, when known
        float dvraw = -1.0f;                            // ... as the batch's table holds it (table position in the low bits)
        float f1x = 0.f, f1y = 0.f, f1z = 0.f;          // first axis
        float f2x = 0.f, f2y = 0.f, f2z = 0.f;          // second axis before orthogonalisation
        unsigned long long n_seen = 0;

        for (int pass = 0; pass < 2; pass++) {
            Best best;
            best.score = -3.0e38f; best.e = 0x7fffffff; best.t = 0x7fffffff;
            float row_lb = -3.0e38f;      // first axis: the best score that some pair of the row is known to reach
            // sweeps: the first axis needs one; the second a first one for the bound and one with the bound
            const int nsweeps = pass == 1 ? 2 : 1;
            for (int sw = 0; sw < nsweeps; sw++) {
                const float bound = (pass == 1 && sw == 1) ? uniform_f(-wave_min(-best.score)) : -3.0e38f;
                for (int pb = 0; pb < npairs; pb += WAVE) {
                    const int npc = min(WAVE, npairs - pb);
                    // stage rpos and q_i.k_j of the pairs, one per lane (a row that fits stays staged for all sweeps;
                    // the pairs of an atom point at consecutive atoms)
                    float4 rq = make_float4(0.f, 0.f, 0.f, 0.f);
                    // (made for the table's box, which every other box of the launch contains: an upper bound there)
                    // (the table's value is rounded down by up to 2^-16 of itself: an upper bound is wanted here)
                    if (sw == 0 && C.pair_near && lane < npc) {
                        dvraw = C.pair_near[e0 + pb + lane].y;
                        dvalid = dvraw * (1.0f + 0x1p-15f);
                    }
                    if (npairs > WAVE || (pass == 0 && sw == 0)) {
                        if (lane < npc) {
                            const int e = e0 + pb + lane;
                            const float4* kp = reinterpret_cast<const float4*>(C.k + ((size_t)(j0 + pb + lane) * H + h) * DH);
                            float qk = 0.0f;
#pragma unroll
                            for (int c4 = 0; c4 < DH / 4; c4++) {
                                const float4 kv = kp[c4];
                                qk = fmaf(qi[4 * c4 + 0], kv.x, qk);
                                qk = fmaf(qi[4 * c4 + 1], kv.y, qk);
                                qk = fmaf(qi[4 * c4 + 2], kv.z, qk);
                                qk = fmaf(qi[4 * c4 + 3], kv.w, qk);
                            }
                            rq = make_float4(P.rpos[(size_t)e * 3 + 0], P.rpos[(size_t)e * 3 + 1],
                                             P.rpos[(size_t)e * 3 + 2], qk);
                        }
                        wave_sync();
                        pq[lane] = rq;
                    } else {
                        rq = pq[lane];
                    }
                    // the noise of a candidate is a hash of (pair, head, pass) shifted by the translation: the hash once per
                    // pair here (three integer multiplications), not once per candidate
                    if (noisy) {
                        wave_sync();
                        sh.ph[lane] = hash_uniform(pass ? seed_hi : seed_lo, pass ? seed_lo : seed_hi,
                                                   (uint32_t)((e0 + pb + lane) * H + h), (uint32_t)pass);
                    }
                    // how far into the sorted table this lane's pair has to look
                    float reach = 3.0e38f;
                    if (a < 0.0f) {
                        const float r2 = fmaf(rq.x, rq.x, fmaf(rq.y, rq.y, rq.z * rq.z));
                        const float r = hw_sqrt(r2);
                        if (sw == 0) {
                            // nearest valid image at distance d: every candidate within the noise of it has
                            // |s| <= |r| + sqrt(d^2 + noise); without the batch's table of d: d <= |r| (+ |s_1|)
                            if (dvalid >= 0.0f) reach = fmaf(1.0001f, r + hw_sqrt(dvalid + nz), 1e-3f);
                            else if (sorted) reach = fmaf(1.0001f, fmaf(2.0f, r, (r2 > 1e-5f ? 0.0f : s1) + sq_nz), 1e-3f);
                        } else if (bound > -1.0e38f) {
                            const float need = (bound - rq.w - 0.5f * nz) * inv_a;
                            reach = need >= 0.0f ? fmaf(1.0001f, r + hw_sqrt(need), 1e-3f) : -1.0f;
                        }
                    }
                    // With the usual box the batch's table names every pair's nearest valid image (d^2 within
                    // [dv_lo, dv_hi], position near_t in the sorted table).
                    const bool near_known = sorted && C.pair_near != nullptr && lane < npc && dvraw >= 0.0f && dvraw < 1.0e37f;
                    const float dv_lo = __uint_as_float(__float_as_uint(dvraw) & ~(uint32_t)(FC_TCAP - 1));
                    const float dv_hi = dv_lo * (1.0f + 0x1p-15f);
                    if (pass == 1 && sw == 0 && sorted && C.pair_near) {
                        // ---- lower bound of the second axis' best score: every pair's nearest valid image, one per lane
                        // (the same arithmetic as in the loop over candidates below, which meets this image again)
                        wave_sync();              // pq (and the phases of the noise) are staged
                        const float4 v = tab[near_known ? (int)(__float_as_uint(dvraw) & (uint32_t)(FC_TCAP - 1)) : 0];
                        const int t = (int)(__float_as_uint(v.w) & (uint32_t)(FC_TCAP - 1));
                        const float dx = rq.x + v.x, dy = rq.y + v.y, dz = rq.z + v.z;
                        const float d2 = fmaf(dx, dx, fmaf(dy, dy, dz * dz));
                        const float rinv = hw_rsq(d2);
                        const float ac = fabsf((dx * f1x + dy * f1y + dz * f1z) * rinv);
                        float score = fmaf(a, d2, rq.w) + hw_log2(fmaxf(1.0f - ac, 1e-5f)) * LN2;
                        if (noisy) {
                            const float un = __builtin_amdgcn_fractf(fmaf((float)t, 0.61803399f, sh.ph[lane]));
                            score += (un - 0.5f) * P.noise;
                        }
                        const int e = e0 + pb + lane;
                        if (near_known && d2 > 1e-5f && ac < 0.9999f && better(score, e, t, best.score, best.e, best.t)) {
                            best.score = score; best.e = e; best.t = t;
                        }
                        n_seen += (unsigned long long)npc;
                        continue;
                    }
                    // First axis: no candidate of a pair scores above hi (its nearest valid image with the noise at its
                    // most favourable), and that image scores at least lo.  A pair whose hi stays below the best lo seen
                    // so far in the row cannot hold the maximum: its candidates are left out.  (The margins cover the
                    // rounding of d^2 in the table of nearest images and of the scores.)
                    bool contender = true;
                    if (pass == 0 && sorted && C.pair_near) {
                        const float hi = near_known ? fmaf(a, dv_lo - 0.5f * nz, rq.w) : 3.0e38f;
                        const float lo_s = near_known ? fmaf(a, dv_hi + 0.5f * nz, rq.w) : -3.0e38f;
                        const float mg = 2e-6f * (fabsf(rq.w) + fabsf(a) * (dv_hi + nz)) + 1e-30f;
                        row_lb = fmaxf(row_lb, uniform_f(wave_maxf(near_known ? lo_s - mg : -3.0e38f)));
                        contender = hi + mg >= row_lb;
                    }
                    for (int ch = 0; ch < nchunks; ch++) {
                        const int t0c = ch * FC_TCAP;
                        const int cnt = sorted ? bx.T : min(FC_TCAP, bx.T - t0c);
                        float4* const tabc = resident ? tab + ch * FC_TCAP : tab;
                        if (nchunks > 1 && !(resident && (pass > 0 || sw > 0 || pb > 0))) {
                            wave_sync();
                            build_sorted_chunk(tabc, t0c, cnt, bx, L, lane);
                        }
                        wave_sync();              // pq, the table; the readers of the marks are done
                        // the bound sweep of the second axis looks at the candidates of the first axis' sweep: when
                        // the row is staged as a whole their list is still there
                        const bool relist = !(pass == 1 && sw == 0 && sorted && npairs <= WAVE);
                        int mine = cnt;           // candidates of this lane's pair: entries with length <= reach
                        if (relist) {
                            int lo = 0, hi = FC_TCAP;
#pragma unroll
                            for (int s = 0; s < 8; s++) {      // the count is one of 0 .. 128: eight halvings
                                const int mid = min((lo + hi) >> 1, FC_TCAP - 1);
                                const bool le = lo < hi && tabc[mid].w <= reach;
                                lo = le ? mid + 1 : lo;
                                hi = le ? hi : mid;
                            }
                            mine = contender ? min(lo, cnt) : 0;
                        }
                        // The candidates of the pairs laid end to end; which pair candidate c belongs to comes without a
                        // search: a bit per candidate marks where the run of a pair begins, so the pair of c is the
                        // number of marks up to c (population counts) into the list of the pairs that have candidates.
                        int total;
                        if (relist) {
                            if (lane >= npc) mine = 0;
                            const int incl = wave_scan_incl(mine);
                            total = __builtin_amdgcn_readlane(incl, WAVE - 1);
                            const int first = incl - mine;
                            const int kslot = (int)lane_prefix(ballot(mine > 0));
#pragma unroll
                            for (int u = 0; u < FC_TCAP / 32; u++) markw[lane + WAVE * u] = 0u;
                            wave_sync();
                            if (mine > 0) {
                                ent[kslot] = (uint32_t)first | ((uint32_t)lane << 16);
                                atomicOr(&markw[first >> 5], 1u << (first & 31));
                            }
                            if (lane == 0) sh.total = total;
                            wave_sync();
                        } else {
                            total = uniform_i(sh.total);
                        }
                        n_seen += (unsigned long long)total;
                        int carry = 0;              // marks in the steps before this one
                        for (int base = 0; base < total; base += WAVE) {
                            const int c = base + lane;
                            const bool in = c < total;
                            const uint64_t m64 = (uint64_t)markw[base >> 5] | ((uint64_t)markw[(base >> 5) + 1] << 32);
                            const int kk = carry + (int)lane_prefix(m64) + (int)((m64 >> lane) & 1ull) - 1;
                            carry += __popcll(m64);
                            const uint32_t en = ent[in ? kk : 0];
                            const int pl = in ? (int)(en >> 16) : 0;
                            const float4 v = tabc[in ? c - (int)(en & 0xffffu) : 0];
                            const float4 cq = pq[pl];
                            const int e = e0 + pb + pl;
                            const int t = t0c + (int)(__float_as_uint(v.w) & (uint32_t)(FC_TCAP - 1));
                            const float dx = cq.x + v.x, dy = cq.y + v.y, dz = cq.z + v.z;
                            const float d2 = fmaf(dx, dx, fmaf(dy, dy, dz * dz));
                            float score = fmaf(a, d2, cq.w);
                            bool ok = in && d2 > 1e-5f;
                            if (pass == 1) {
                                const float rinv = hw_rsq(d2);
                                const float ac = fabsf((dx * f1x + dy * f1y + dz * f1z) * rinv);
                                score += hw_log2(fmaxf(1.0f - ac, 1e-5f)) * LN2;
                                ok = ok && ac < 0.9999f;
                            }
                            if (noisy) {
                                const float phase = sh.ph[pl];
                                const float un = __builtin_amdgcn_fractf(fmaf((float)t, 0.61803399f, phase));
                                if (pass == 0) score = fmaf(a, d2 + (un - 0.5f) * P.noise, cq.w);
                                else score += (un - 0.5f) * P.noise;
                            }
                            if (ok && better(score, e, t, best.score, best.e, best.t)) {
                                best.score = score; best.e = e; best.t = t;
                            }
                        }
                    }
                }
            }
            wave_best(best);
            float vx = 0.f, vy = 0.f, vz = 0.f;
            if (best.e != 0x7fffffff) {
                float sx, sy, sz;
                shift_of(best.t, bx, L, sx, sy, sz);
                if (npairs <= WAVE) {                 // the row is still staged
                    const float4 rq = pq[best.e - e0];
                    vx = rq.x + sx; vy = rq.y + sy; vz = rq.z + sz;
                } else {
                    vx = uniform_f(P.rpos[(size_t)best.e * 3 + 0]) + sx;
                    vy = uniform_f(P.rpos[(size_t)best.e * 3 + 1]) + sy;
                    vz = uniform_f(P.rpos[(size_t)best.e * 3 + 2]) + sz;
                }
                unit_vector(vx, vy, vz);
            }
            if (pass == 0) { f1x = vx; f1y = vy; f1z = vz; }
            else { f2x = vx; f2y = vy; f2z = vz; }
        }

        if (lane == 0) {
            float gx, gy, gz, hx, hy, hz;
            orthonormal_axes(f1x, f1y, f1z, f2x, f2y, f2z, gx, gy, gz, hx, hy, hz);
            const size_t stride = (size_t)P.N * H * 3;
            float* o = P.out_frame + ((size_t)i * H + h) * 3;
            o[0] = f1x; o[1] = f1y; o[2] = f1z;
            o[stride + 0] = gx; o[stride + 1] = gy; o[stride + 2] = gz;
            o[2 * stride + 0] = hx; o[2 * stride + 1] = hy; o[2 * stride + 2] = hz;
            if (P.frames_to_records) {
                // the record of this item becomes that of the kernel that follows: the query makes room for the frames
                float* r = reinterpret_cast<float*>(P.items + ((size_t)it_cur * H + h) * REC_WORDS + REC_FRAMES);
                r[0] = f1x; r[1] = f1y; r[2] = f1z;
                r[3] = gx; r[4] = gy; r[5] = gz;
                r[6] = hx; r[7] = hy; r[8] = hz;
            }
        }
        if (P.stats && lane == 0) atomicAdd(P.stats + STAT_FRAME1_RAW, n_seen);      // candidates looked at, both axes
    }
}

// ---- four heads of one atom per wavefront ----------------------------------------------------------------------
// The items (atom, head) of an atom share everything but the query, the Gaussian coefficient and therefore the
// scores: same pairs, same sorted table, same distances.  One wavefront takes four heads of an atom, one per
// 16-lane row.  The pairs are staged once for all four rows (positions and nearest-image distances, and q.k per head);
// every row then lays its own candidates end to end and deals them to its 16 lanes, and keeps its own best.  The
// loops run as long as the longest row needs (the four rows have the same pairs, so nearly the same lengths);
// reductions stay inside a row (DPP).  Compared with one wavefront per item: a quarter of the staging work per item,
// lanes filled by four short candidate lists instead of one, four independent items in flight per wavefront.
// Rows whose box is not the table's are left to frame_axes_sorted_kernel (unsorted_only).
template <int CTRL>
__device__ __forceinline__ float row_maxf_step(float x) { return fmaxf(x, dpp_move<CTRL>(x)); }
__device__ __forceinline__ float row_max(float x) {
    x = row_maxf_step<0xB1>(x); x = row_maxf_step<0x4E>(x); x = row_maxf_step<0x141>(x); x = row_maxf_step<0x140>(x);
    return x;
}
__device__ __forceinline__ void row_best(Best& b) {
    best_dpp<0xB1>(b); best_dpp<0x4E>(b); best_dpp<0x141>(b); best_dpp<0x140>(b);
}

struct FrameQuadShared {
    float4 tab[FC_TCAP];
    float4 rp[FQ_STAGE];                 // staged pairs: rpos, d^2 of the nearest valid image (or -1)
    float qk_s[FQ_ROWS][FQ_STAGE];       // q_h . k_j of the staged pairs, per row
    float ph_s[2][FQ_ROWS][FQ_STAGE];    // phase of the tie-breaking noise of the staged pairs, per pass and row
    uint32_t markw[FQ_ROWS][FQ_PAIR_GROUP * FC_TCAP / 32];      // per row: one bit per candidate, set where a pair's run begins
    uint32_t ent[FQ_ROWS][16];           // per row: the pairs that have candidates, in order: first candidate | pair << 16
};
// one wavefront, four heads of one atom: wid = item * groups + group of heads
__device__ __forceinline__ void frame_quad_body(const CoreArgs& C, FrameQuadShared& sh, int wid, int lane) {
    float4* const tab = sh.tab;
    float4* const rp = sh.rp;
    float (*const qk_s)[FQ_STAGE] = sh.qk_s;
    uint32_t (*const markw)[FQ_PAIR_GROUP * FC_TCAP / 32] = sh.markw;
    uint32_t (*const ent)[16] = sh.ent;

    const KernelArgs& P = C.K;
    const int row = lane >> 4, l16 = lane & 15;
    const int H = P.H;
    const int groups = (H + FQ_ROWS - 1) / FQ_ROWS;
    // (groups of heads: a power of two for 4, 8, 16 ... heads, then without a division)
    const bool pow2 = (groups & (groups - 1)) == 0;
    const int it = pow2 ? wid >> (__ffs(groups) - 1) : wid / groups, hg = wid - it * groups;
    if (it >= P.N) return;
    const int h_row = min(hg * FQ_ROWS + row, H - 1);
    const bool row_exists = hg * FQ_ROWS + row < H;
    const bool noisy = P.noise > 0.0f;
    uint32_t seed_lo = P.seed_lo, seed_hi = P.seed_hi;
    if (noisy && P.seed_dev) {
        const unsigned long long s = *P.seed_snap;
        seed_lo ^= (uint32_t)s * 0x9E3779B1u;
        seed_hi += (uint32_t)(s >> 32) ^ ((uint32_t)s * 0x85EBCA77u);
    }
    // record of this row's item: atom, pairs, lattice, first neighbour and crystal are the same in all four
    const uint32_t* rec = P.items + ((size_t)it * H + h_row) * REC_WORDS;
    const uint32_t w0 = rec[l16], w1 = rec[16 + l16];
    const int i = __builtin_amdgcn_readlane((int)w0, REC_ATOM);
    const int e0 = __builtin_amdgcn_readlane((int)w0, REC_E0);
    const int npairs = __builtin_amdgcn_readlane((int)w0, REC_NPAIRS);
    const int j0 = __builtin_amdgcn_readlane((int)w1, REC_J0 - 16);
    const int crystal = __builtin_amdgcn_readlane((int)w1, REC_CRYSTAL - 16);
    Lattice L;
#pragma unroll
    for (int d = 0; d < 9; d++) L.t[d] = __int_as_float(__builtin_amdgcn_readlane((int)w0, REC_LATTICE + d));
    const int boxw = (int)rec[REC_BOX];
    const float a = __uint_as_float(rec[REC_A]);
    const float inv_a = a < 0.0f ? hw_rcp(a) : 0.0f;      // (for a reach with margins: the hardware reciprocal will do)
    float q[DH];
    {
        const float4* qp = reinterpret_cast<const float4*>(rec + REC_QUERY);
#pragma unroll
        for (int c4 = 0; c4 < DH / 4; c4++) {
            const float4 v = qp[c4];
            q[4 * c4] = v.x; q[4 * c4 + 1] = v.y; q[4 * c4 + 2] = v.z; q[4 * c4 + 3] = v.w;
        }
    }
    const int R0 = C.table_R;
    // this row is searched here (the others by frame_item_body)
    const bool mine = row_exists && boxw == (R0 | (R0 << 8) | (R0 << 16)) && a < 0.0f && npairs <= FQ_MAX_PAIRS;
    if (ballot(mine) == 0) return;
    Box bx;
    bx.R1 = bx.R2 = bx.R3 = R0; bx.s2 = bx.s3 = 2 * R0 + 1; bx.T = bx.s2 * bx.s2 * bx.s2; bx.over = 0;
    {
        const float4* src = C.sorted_tab + (size_t)crystal * FC_TCAP;
        tab[lane] = src[lane];
        tab[lane + WAVE] = src[lane + WAVE];
    }
    const float nz = noisy ? P.noise : 0.0f;
    const float sq_nz = sqrtf(nz);
    wave_sync();
    const float s1 = tab[1].w;          // shortest non-zero shift (entry 0 is the zero shift)

    float f1x = 0.f, f1y = 0.f, f1z = 0.f, f2x = 0.f, f2y = 0.f, f2z = 0.f;
    unsigned long long n_seen = 0;
    for (int pass = 0; pass < 2; pass++) {
        Best best;
        best.score = -3.0e38f; best.e = 0x7fffffff; best.t = 0x7fffffff;
        for (int sw = 0; sw < (pass == 1 ? 2 : 1); sw++) {
            const float bound = (pass == 1 && sw == 1) ? row_max(best.score) : -3.0e38f;      // per row
            for (int pb = 0; pb < npairs; pb += FQ_STAGE) {
                const int nst = min(FQ_STAGE, npairs - pb);
                if (npairs > FQ_STAGE || (pass == 0 && sw == 0)) {
                    // ---- stage: lane = pair; q.k for the four heads with the query channels read across the rows
                    wave_sync();
                    float4 r4 = make_float4(0.f, 0.f, 0.f, -1.0f);
                    const bool have = lane < nst;
                    const int e = e0 + pb + min(lane, nst - 1);
                    if (have) {
                        r4.x = P.rpos[(size_t)e * 3 + 0]; r4.y = P.rpos[(size_t)e * 3 + 1]; r4.z = P.rpos[(size_t)e * 3 + 2];
                        if (C.pair_near) r4.w = C.pair_near[e].y;
                    }
                    if (lane < FQ_STAGE) rp[lane] = r4;
#pragma unroll 1
                    for (int r = 0; r < FQ_ROWS; r++) {
                        const int hr = min(hg * FQ_ROWS + r, H - 1);
                        const float4* kp = reinterpret_cast<const float4*>(C.k + ((size_t)(j0 + pb + min(lane, nst - 1)) * H + hr) * DH);
                        float acc = 0.0f;
#pragma unroll
                        for (int c4 = 0; c4 < DH / 4; c4++) {
                            const float4 kv = kp[c4];
                            acc = fmaf(__int_as_float(__builtin_amdgcn_readlane(__float_as_int(q[4 * c4 + 0]), r * 16)), kv.x, acc);
                            acc = fmaf(__int_as_float(__builtin_amdgcn_readlane(__float_as_int(q[4 * c4 + 1]), r * 16)), kv.y, acc);
                            acc = fmaf(__int_as_float(__builtin_amdgcn_readlane(__float_as_int(q[4 * c4 + 2]), r * 16)), kv.z, acc);
                            acc = fmaf(__int_as_float(__builtin_amdgcn_readlane(__float_as_int(q[4 * c4 + 3]), r * 16)), kv.w, acc);
                        }
                        if (lane < FQ_STAGE) qk_s[r][lane] = acc;
                    }
                    // the noise of a candidate is a hash of (pair, head, pass) shifted by the translation: the hash once per
                    // pair and pass here (three integer multiplications), not once per candidate
                    if (noisy) {
                        const uint32_t key = (uint32_t)((e0 + pb + min(l16, nst - 1)) * H + h_row);
                        sh.ph_s[0][row][l16] = hash_uniform(seed_lo, seed_hi, key, 0u);
                        sh.ph_s[1][row][l16] = hash_uniform(seed_hi, seed_lo, key, 1u);
                    }
                    wave_sync();
                }
                for (int pc = 0; pc < nst; pc += 16) {
                    // ---- this row's 16 pairs: how far each has to look, its candidates end to end
                    const int pj = pc + l16;
                    const bool pair_ok = mine && pj < nst;
                    const float4 r4 = rp[min(pj, nst - 1)];
                    const float myqk = qk_s[row][min(pj, nst - 1)];
                    const float r2 = fmaf(r4.x, r4.x, fmaf(r4.y, r4.y, r4.z * r4.z));
                    const float r = hw_sqrt(r2);
                    // the pair's nearest valid image, when the batch's table of them is there: its d^2 lies in
                    // [dv_lo, dv_hi], its position in the sorted table is near_t
                    const bool near_known = r4.w >= 0.0f && r4.w < 1.0e37f;
                    const float dv_lo = __uint_as_float(__float_as_uint(r4.w) & ~(uint32_t)(FC_TCAP - 1));
                    const float dv_hi = dv_lo * (1.0f + 0x1p-15f);
                    const int near_t = (int)(__float_as_uint(r4.w) & (uint32_t)(FC_TCAP - 1));
                    if (pass == 1 && sw == 0 && C.pair_near) {
                        // ---- lower bound of the second axis' best score: every pair's nearest valid image, one per lane
                        // (the same arithmetic as in the loop over candidates below, which meets this image again)
                        const float4 v = tab[near_known ? near_t : 0];
                        const int t = (int)(__float_as_uint(v.w) & (uint32_t)(FC_TCAP - 1));
                        const float dx = r4.x + v.x, dy = r4.y + v.y, dz = r4.z + v.z;
                        const float d2 = fmaf(dx, dx, fmaf(dy, dy, dz * dz));
                        const float rinv = hw_rsq(d2);
                        const float ac = fabsf((dx * f1x + dy * f1y + dz * f1z) * rinv);
                        float score = fmaf(a, d2, myqk) + hw_log2(fmaxf(1.0f - ac, 1e-5f)) * LN2;
                        if (noisy) {
                            const float phase = sh.ph_s[1][row][min(pj, nst - 1)];
                            const float un = __builtin_amdgcn_fractf(fmaf((float)t, 0.61803399f, phase));
                            score += (un - 0.5f) * P.noise;
                        }
                        const int e = e0 + pb + pj;
                        if (pair_ok && near_known && d2 > 1e-5f && ac < 0.9999f && better(score, e, t, best.score, best.e, best.t)) {
                            best.score = score; best.e = e; best.t = t;
                        }
                        n_seen += (unsigned long long)__popcll(ballot(pair_ok));
                        continue;
                    }
                    float reach;
                    if (sw == 0) {
                        reach = near_known ? fmaf(1.0001f, r + hw_sqrt(dv_hi + nz), 1e-3f)
                                           : fmaf(1.0001f, fmaf(2.0f, r, (r2 > 1e-5f ? 0.0f : s1) + sq_nz), 1e-3f);
                    } else if (bound > -1.0e38f) {
                        const float need = (bound - myqk - 0.5f * nz) * inv_a;
                        reach = need >= 0.0f ? fmaf(1.0001f, r + hw_sqrt(need), 1e-3f) : -1.0f;
                    } else {
                        reach = 3.0e38f;
                    }
                    int cnt;
                    {
                        int lo = 0, hi = FC_TCAP;
#pragma unroll
                        for (int s = 0; s < 8; s++) {      // the count is one of 0 .. 128: eight halvings
                            const int mid = min((lo + hi) >> 1, FC_TCAP - 1);
                            const bool le = lo < hi && tab[mid].w <= reach;
                            lo = le ? mid + 1 : lo;
                            hi = le ? hi : mid;
                        }
                        cnt = pair_ok ? min(lo, bx.T) : 0;
                    }
                    if (pass == 0 && C.pair_near) {
                        // First axis: no candidate of a pair scores above hi (its nearest valid image with the noise at
                        // its most favourable), and its nearest valid image scores at least lo.  A pair whose hi stays
                        // below the best lo of the row cannot hold the maximum: its candidates are left out.  (The
                        // margins cover the rounding of d^2 in the table of nearest images and of the scores.)
                        const float hi = near_known ? fmaf(a, dv_lo - 0.5f * nz, myqk) : 3.0e38f;
                        const float lo_s = near_known ? fmaf(a, dv_hi + 0.5f * nz, myqk) : -3.0e38f;
                        const float mg = 2e-6f * (fabsf(myqk) + fabsf(a) * (dv_hi + nz)) + 1e-30f;
                        const float lb = row_max(pair_ok ? lo_s - mg : -3.0e38f);
                        if (!(hi + mg >= lb)) cnt = 0;
                    }
                    int incl = cnt;                        // inclusive prefix within the row
                    incl += dpp_movei<0x111>(incl);
                    incl += dpp_movei<0x112>(incl);
                    incl += dpp_movei<0x114>(incl);
                    incl += dpp_movei<0x118>(incl);
                    const int t0 = __builtin_amdgcn_readlane(incl, 15), t1 = __builtin_amdgcn_readlane(incl, 31);
                    const int t2 = __builtin_amdgcn_readlane(incl, 47), t3 = __builtin_amdgcn_readlane(incl, 63);
                    const int total = row == 0 ? t0 : row == 1 ? t1 : row == 2 ? t2 : t3;
                    const int longest = max(max(t0, t1), max(t2, t3));
                    // Which pair a candidate belongs to, without a search: a bit per candidate marks where the run of a
                    // pair begins, so the pair of candidate c is the number of marks up to c (a population count of
                    // the 16 marks of the step plus what the steps before counted) into the list of the pairs that
                    // have candidates.  One read of the marks and one of that list per step, instead of four dependent
                    // reads of a bisection: the step's latency was what the wavefronts waited for.
                    const uint32_t nzrow = (uint32_t)(ballot(cnt > 0) >> (16 * row)) & 0xffffu;
                    const int kslot = __popc(nzrow & ((1u << l16) - 1u));
                    const int first = incl - cnt;
                    wave_sync();                           // the readers of the marks and the list are done
#pragma unroll
                    for (int u = 0; u < FQ_PAIR_GROUP * FC_TCAP / 32 / 16; u++) markw[row][l16 + 16 * u] = 0u;
                    wave_sync();
                    if (cnt > 0) {
                        ent[row][kslot] = (uint32_t)first | ((uint32_t)l16 << 16);
                        atomicOr(&markw[row][first >> 5], 1u << (first & 31));
                    }
                    wave_sync();
                    n_seen += (unsigned long long)(t0 + t1 + t2 + t3);
                    int carry = 0;                         // marks in the steps before this one (the same in a row)
                    for (int base = 0; base < longest; base += 16) {
                        const int c = base + l16;
                        const bool in = c < total;
                        const uint32_t m16 = (markw[row][base >> 5] >> (base & 16)) & 0xffffu;
                        const int kk = carry + __popc(m16 & ((2u << l16) - 1u)) - 1;
                        carry += __popc(m16);
                        const uint32_t en = ent[row][in ? kk : 0];
                        const int pl = in ? (int)(en >> 16) : 0;
                        const float4 v = tab[in ? c - (int)(en & 0xffffu) : 0];
                        const int ps = min(pc + pl, nst - 1);
                        const float4 cq = rp[ps];
                        const float cqk = qk_s[row][ps];
                        const int e = e0 + pb + pc + pl;
                        const int t = (int)(__float_as_uint(v.w) & (uint32_t)(FC_TCAP - 1));
                        const float dx = cq.x + v.x, dy = cq.y + v.y, dz = cq.z + v.z;
                        const float d2 = fmaf(dx, dx, fmaf(dy, dy, dz * dz));
                        float score = fmaf(a, d2, cqk);
                        bool ok = in && d2 > 1e-5f;
                        if (pass == 1) {
                            const float rinv = hw_rsq(d2);
                            const float ac = fabsf((dx * f1x + dy * f1y + dz * f1z) * rinv);
                            score += hw_log2(fmaxf(1.0f - ac, 1e-5f)) * LN2;
                            ok = ok && ac < 0.9999f;
                        }
                        if (noisy) {
                            const float phase = sh.ph_s[pass][row][ps];
                            const float un = __builtin_amdgcn_fractf(fmaf((float)t, 0.61803399f, phase));
                            if (pass == 0) score = fmaf(a, d2 + (un - 0.5f) * P.noise, cqk);
                            else score += (un - 0.5f) * P.noise;
                        }
                        if (ok && better(score, e, t, best.score, best.e, best.t)) {
                            best.score = score; best.e = e; best.t = t;
                        }
                    }
                }
            }
        }
        row_best(best);
        float vx = 0.f, vy = 0.f, vz = 0.f;
        if (best.e != 0x7fffffff) {
            float sx, sy, sz;
            shift_of(best.t, bx, L, sx, sy, sz);
            vx = P.rpos[(size_t)best.e * 3 + 0] + sx;
            vy = P.rpos[(size_t)best.e * 3 + 1] + sy;
            vz = P.rpos[(size_t)best.e * 3 + 2] + sz;
            unit_vector(vx, vy, vz);
        }
        if (pass == 0) { f1x = vx; f1y = vy; f1z = vz; }
        else { f2x = vx; f2y = vy; f2z = vz; }
    }
    // lane c < 9 of a row stores component c of that row's frame
    float gx, gy, gz, hx, hy, hz;
    orthonormal_axes(f1x, f1y, f1z, f2x, f2y, f2z, gx, gy, gz, hx, hy, hz);
    if (mine && l16 < 9) {
        const float val = l16 == 0 ? f1x : l16 == 1 ? f1y : l16 == 2 ? f1z : l16 == 3 ? gx : l16 == 4 ? gy : l16 == 5 ? gz
                        : l16 == 6 ? hx : l16 == 7 ? hy : hz;
        const int ax = l16 / 3, d = l16 - 3 * ax;
        P.out_frame[(((size_t)ax * P.N + i) * H + h_row) * 3 + d] = val;
        if (P.frames_to_records)      // the record becomes that of the kernel that follows: the query makes room for the frames
            reinterpret_cast<float*>(P.items + ((size_t)it * H + h_row) * REC_WORDS + REC_FRAMES)[l16] = val;
    }
    if (P.stats && lane == 0) atomicAdd(P.stats + STAT_FRAME1_RAW, n_seen);
}

// One item per wavefront, every item (launches without per-crystal tables).  waves: N * H.
__global__ __launch_bounds__(WAVE * CORE_WPB) void frame_axes_sorted_kernel(const CoreArgs C) {
    __shared__ FrameShared shared[CORE_WPB];
    frame_item_body(C, shared[threadIdx.x >> 6], (int)blockIdx.x * CORE_WPB + (int)(threadIdx.x >> 6),
                    (int)threadIdx.x & (WAVE - 1), false, false);
}

// Both ways in one launch, the slowest work first.  Wavefronts in the order of the grid:
//   1. one per listed record with a box of their own, by rank over the lists (made by the launch that wrote the
//      records; no record of that rank: the wavefront ends): several sorted chunks, the longest of the launch;
//   2. the four-heads search over all atoms;
//   3. one per item, for the items that neither of the two takes (usual box, longer rows: they are at the start of the
//      work order, so the wavefronts that find nothing to do come last and only pass through).
// With the items of (3) and their many passing wavefronts in front, the four-heads search started after a third of
// the launch's time, and the records with a box of their own, scattered over the work order, later still.
__global__ __launch_bounds__(WAVE * CORE_WPB) void frame_axes_kernel(const CoreArgs C, int slow_blocks, int quad_blocks) {
    __shared__ union { FrameShared item; FrameQuadShared quad; } shared[CORE_WPB];
    const int wv = (int)(threadIdx.x >> 6), lane = (int)threadIdx.x & (WAVE - 1);
    const int blk = (int)blockIdx.x;
    if (blk >= slow_blocks && blk < slow_blocks + quad_blocks) {
        frame_quad_body(C, shared[wv].quad, (blk - slow_blocks) * CORE_WPB + wv, lane);
        return;
    }
    const bool listed = blk < slow_blocks;
    const int wid = listed ? core_slow_record(C, blk * CORE_WPB + wv, lane) : (blk - slow_blocks - quad_blocks) * CORE_WPB + wv;
    if (wid < 0) return;
    frame_item_body(C, shared[wv].item, wid, lane, !listed, !listed && slow_blocks > 0);
}

}  // namespace cfh
