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
//   * second axis: score = q.k + a d^2 + log(max(1 - |cos|, 1e-5)) <= q.k + a d^2.  A first sweep over the same
//     prefixes gives a lower bound `best` of the maximum; a candidate of pair j can then only matter if
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

// shifts t0 .. t0+cnt of the box in the reference's loop order, w = position in the chunk (read like the low bits of
// the sorted table's packed length: a tiny value that passes every reach test)
__device__ __forceinline__ void build_shift_table_indexed(float4* tab, int t0, int cnt, const Box& bx, const Lattice& L,
                                                          int lane) {
    for (int u = lane; u < cnt; u += WAVE) {
        const int t = t0 + u;
        const int i3 = t % bx.s3;
        const int q = t / bx.s3;
        const int i2 = q % bx.s2;
        const int i1 = q / bx.s2;
        const float n1 = (float)(i1 - bx.R1), n2 = (float)(i2 - bx.R2), n3 = (float)(i3 - bx.R3);
        float4 v;
        v.x = fmaf(L.t[6], n3, fmaf(L.t[3], n2, L.t[0] * n1));
        v.y = fmaf(L.t[7], n3, fmaf(L.t[4], n2, L.t[1] * n1));
        v.z = fmaf(L.t[8], n3, fmaf(L.t[5], n2, L.t[2] * n1));
        v.w = __uint_as_float((uint32_t)u);
        tab[u] = v;
    }
}

// inclusive prefix sum over the 64 lanes (row scans in DPP, row totals by lane reads)
__device__ __forceinline__ int wave_scan_incl(int x) {
    x += dpp_movei<0x111>(x);
    x += dpp_movei<0x112>(x);
    x += dpp_movei<0x114>(x);
    x += dpp_movei<0x118>(x);
    const int t0 = __builtin_amdgcn_readlane(x, 15), t1 = __builtin_amdgcn_readlane(x, 31);
    const int t2 = __builtin_amdgcn_readlane(x, 47);
    const int row = (int)threadIdx.x >> 4;
    return x + (row == 0 ? 0 : row == 1 ? t0 : row == 2 ? t0 + t1 : t0 + t1 + t2);
}

__global__ __launch_bounds__(WAVE) void frame_axes_sorted_kernel(const CoreArgs C) {
    __shared__ float4 tab[FC_TCAP];
    __shared__ float4 pq[WAVE];             // rpos and q.k of the staged pairs
    __shared__ int pstart[WAVE + 1];        // first candidate of every staged pair, then the total

    const KernelArgs& P = C.K;
    const int lane = threadIdx.x;
    const int H = P.H;
    const int h = blockIdx.x % H;
    const bool noisy = P.noise > 0.0f;
    uint32_t seed_lo = P.seed_lo, seed_hi = P.seed_hi;
    if (noisy && P.seed_dev) {
        const unsigned long long s = *P.seed_snap;
        seed_lo ^= (uint32_t)s * 0x9E3779B1u;
        seed_hi += (uint32_t)(s >> 32) ^ ((uint32_t)s * 0x85EBCA77u);
    }

    const int it_cur = (int)blockIdx.x / H;      // one wavefront per item, long items first
    if (it_cur >= P.N) return;
    {
        const uint32_t rec_cur = load_record(P, it_cur, h);
        const Item item = unpack_item(rec_cur);
        const int crystal = __builtin_amdgcn_readlane((int)rec_cur, REC_CRYSTAL);
        const int j0 = __builtin_amdgcn_readlane((int)rec_cur, REC_J0);
        const int i = item.i;
        const float a = item.a;
        const Lattice L = item.L;
        const Box bx = item.bx;
        float qi[DH];
#pragma unroll
        for (int c = 0; c < DH; c++) qi[c] = rec_f(rec_cur, REC_QUERY + c);
        const bool sorted = C.sorted_tab != nullptr && bx.R1 == C.table_R && bx.R2 == C.table_R && bx.R3 == C.table_R &&
                            a < 0.0f;
        const int nchunks = sorted ? 1 : (bx.T + FC_TCAP - 1) / FC_TCAP;
        const int e0 = item.e0, npairs = item.npairs;
        const float nz = noisy ? P.noise : 0.0f;
        const float sq_nz = sqrtf(nz);

        if (sorted) {
            const float4* src = C.sorted_tab + (size_t)crystal * FC_TCAP;
            tab[lane] = src[lane];
            tab[lane + WAVE] = src[lane + WAVE];
        } else if (nchunks == 1) {
            build_shift_table_indexed(tab, 0, bx.T, bx, L, lane);
        }
        wave_sync();
        const float s1 = sorted ? tab[1].w : 0.0f;      // shortest non-zero shift (entry 0 is the zero shift)

        float dvalid = -1.0f;                           // this lane's pair: d^2 of its nearest valid image, when known
        float f1x = 0.f, f1y = 0.f, f1z = 0.f;          // first axis
        float f2x = 0.f, f2y = 0.f, f2z = 0.f;          // second axis before orthogonalisation
        unsigned long long n_seen = 0;

        for (int pass = 0; pass < 2; pass++) {
            Best best;
            best.score = -3.0e38f; best.e = 0x7fffffff; best.t = 0x7fffffff;
            // sweeps: the first axis needs one; the second a first one for the bound and one with the bound
            const int nsweeps = (pass == 1 && sorted) ? 2 : 1;
            for (int sw = 0; sw < nsweeps; sw++) {
                const float bound = (pass == 1 && sw == 1) ? uniform_f(-wave_min(-best.score)) : -3.0e38f;
                for (int pb = 0; pb < npairs; pb += WAVE) {
                    const int npc = min(WAVE, npairs - pb);
                    // stage rpos and q_i.k_j of the pairs, one per lane (a row that fits stays staged for all sweeps;
                    // the pairs of an atom point at consecutive atoms)
                    float4 rq = make_float4(0.f, 0.f, 0.f, 0.f);
                    if (sw == 0 && C.pair_near && sorted && lane < npc) dvalid = C.pair_near[e0 + pb + lane].y;
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
                    // how far into the sorted table this lane's pair has to look
                    float reach = 3.0e38f;
                    if (sorted) {
                        const float r2 = fmaf(rq.x, rq.x, fmaf(rq.y, rq.y, rq.z * rq.z));
                        const float r = hw_sqrt(r2);
                        if (sw == 0) {
                            // nearest valid image at distance d: every candidate within the noise of it has
                            // |s| <= |r| + sqrt(d^2 + noise); without the batch's table of d: d <= |r| (+ |s_1|)
                            reach = dvalid >= 0.0f ? fmaf(1.0001f, r + hw_sqrt(dvalid + nz), 1e-3f)
                                                   : fmaf(1.0001f, fmaf(2.0f, r, (r2 > 1e-5f ? 0.0f : s1) + sq_nz), 1e-3f);
                        } else if (bound > -1.0e38f) {
                            const float need = (bound - rq.w - 0.5f * nz) / a;
                            reach = need >= 0.0f ? fmaf(1.0001f, r + hw_sqrt(need), 1e-3f) : -1.0f;
                        }
                    }
                    for (int ch = 0; ch < nchunks; ch++) {
                        const int t0c = ch * FC_TCAP;
                        const int cnt = sorted ? bx.T : min(FC_TCAP, bx.T - t0c);
                        if (nchunks > 1) {
                            wave_sync();
                            build_shift_table_indexed(tab, t0c, cnt, bx, L, lane);
                        }
                        wave_sync();              // pq, the table; the readers of pstart are done
                        // the bound sweep of the second axis looks at the candidates of the first axis' sweep: when
                        // the row is staged as a whole their list is still there
                        const bool relist = !(pass == 1 && sw == 0 && sorted && npairs <= WAVE);
                        int mine = cnt;           // candidates of this lane's pair: entries with length <= reach
                        if (sorted && relist) {
                            int lo = 0, hi = FC_TCAP;
#pragma unroll
                            for (int s = 0; s < 8; s++) {      // the count is one of 0 .. 128: eight halvings
                                const int mid = min((lo + hi) >> 1, FC_TCAP - 1);
                                const bool le = lo < hi && tab[mid].w <= reach;
                                lo = le ? mid + 1 : lo;
                                hi = le ? hi : mid;
                            }
                            mine = min(lo, cnt);
                        }
                        int total;
                        if (relist) {
                            if (lane >= npc) mine = 0;
                            const int incl = wave_scan_incl(mine);
                            total = __builtin_amdgcn_readlane(incl, WAVE - 1);
                            pstart[lane] = incl - mine;
                            if (lane == 0) pstart[WAVE] = total;
                            wave_sync();
                        } else {
                            total = uniform_i(pstart[WAVE]);
                        }
                        n_seen += (unsigned long long)total;

                        for (int base = 0; base < total; base += WAVE) {
                            const int c = base + lane;
                            const bool in = c < total;
                            int lo = 0, hi = WAVE;      // pstart[lo] <= c < pstart[hi]
#pragma unroll
                            for (int s = 0; s < 6; s++) {
                                const int mid = (lo + hi) >> 1;
                                const bool le = pstart[mid] <= c;
                                lo = le ? mid : lo;
                                hi = le ? hi : mid;
                            }
                            const int pl = in ? lo : 0;
                            const float4 v = tab[in ? c - pstart[pl] : 0];
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
                                const float phase = hash_uniform(pass ? seed_hi : seed_lo, pass ? seed_lo : seed_hi,
                                                                 (uint32_t)(e * H + h), (uint32_t)pass);
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
                const float inv = 1.0f / sqrtf(vx * vx + vy * vy + vz * vz);
                vx *= inv; vy *= inv; vz *= inv;
            }
            if (pass == 0) { f1x = vx; f1y = vy; f1z = vz; }
            else { f2x = vx; f2y = vy; f2z = vz; }
        }

        if (lane == 0) {
            // Gram-Schmidt and cross product
            // (models/indexed_lattice_multi_head_attention_cuda.py:475-481; F.normalize eps 1e-12)
            const float dot = f1x * f2x + f1y * f2y + f1z * f2z;
            float gx = f2x - dot * f1x, gy = f2y - dot * f1y, gz = f2z - dot * f1z;
            const float inv = 1.0f / fmaxf(sqrtf(gx * gx + gy * gy + gz * gz), 1e-12f);
            gx *= inv; gy *= inv; gz *= inv;
            const size_t stride = (size_t)P.N * H * 3;
            float* o = P.out_frame + ((size_t)i * H + h) * 3;
            o[0] = f1x; o[1] = f1y; o[2] = f1z;
            o[stride + 0] = gx; o[stride + 1] = gy; o[stride + 2] = gz;
            const float hx = f1y * gz - f1z * gy, hy = f1z * gx - f1x * gz, hz = f1x * gy - f1y * gx;
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

}  // namespace cfh
