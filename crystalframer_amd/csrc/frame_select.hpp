// Dynamic "max" frame selection.  For every (atom i, head h) the first axis points to the most
// attended periodic image, the second (before orthogonalisation) to the image maximising the
// attention logit plus log(1-|cos|) to the first axis.  One wavefront scans all neighbours j and
// all translations n of an (i,h) item and keeps the joint arg-max, which replaces the reference's
// per-edge kernel + gathered q.k product + third-party segmented arg-max
// (models/kernels/compute_maximum_frame_each_edge.cu:78-111,
//  models/kernels/compute_second_frame_each_edge.cu:81-142,
//  models/cuda_funcs/calc_maximum_frame.py:72-86,146-164).
//
// Both searches are arg-maxima over (j, n) of one expression -- q_i.k_j + a d^2 for the first axis
// (for a < 0 the nearest image of a neighbour is also its best), q_i.k_j + a d^2 + log(max(1-|cos|,
// 1e-5)) for the second -- so every lane keeps a running best over its own translations of every
// pair and the wavefront reduces once per item.  Tie rule with zero noise: lowest pair index, then
// first translation in the reference's loop order (what its strict comparisons and the plain
// arg-max over pairs give).  With noise > 0 every candidate's key is perturbed by a uniform in
// (-noise/2, noise/2): a golden-ratio sequence over the translations with a hashed phase per
// (pair, head, pass, seed) -- three operations per candidate (the reference draws from cuRAND
// XORWOW seeded by numpy; its stream cannot be reproduced, only its distribution).
//
// MODE 0: first axis only.  MODE 1: second axis for a given first axis.  MODE 2: both, then
// Gram-Schmidt and the cross product, written as (3,N,H,3) orthonormal frames.
#pragma once
#include "device_common.hpp"

namespace cfh {

// translation index -> box coordinates, t = (i1 s2 + i2) s3 + i3; the quotients by float reciprocal
// (exact: t + 1/2 over a divisor below 2^10 is never within rounding of an integer)
__device__ __forceinline__ void box_coords(int t, const Box& bx, float inv_s2, float inv_s3, int& n1, int& n2, int& n3) {
    const int q = (int)(((float)t + 0.5f) * inv_s3);
    const int i1 = (int)(((float)q + 0.5f) * inv_s2);
    n3 = t - q * bx.s3 - bx.R3;
    n2 = q - i1 * bx.s2 - bx.R2;
    n1 = i1 - bx.R1;
}
__device__ __forceinline__ void shift_of(int t, const Box& bx, const Lattice& L, float& vx, float& vy,
                                         float& vz) {
    int m1, m2, m3;
    box_coords(t, bx, hw_rcp((float)bx.s2), hw_rcp((float)bx.s3), m1, m2, m3);      // (within an ulp: the quotients stay exact)
    const float n1 = (float)m1, n2 = (float)m2, n3 = (float)m3;
    vx = fmaf(L.t[6], n3, fmaf(L.t[3], n2, L.t[0] * n1));
    vy = fmaf(L.t[7], n3, fmaf(L.t[4], n2, L.t[1] * n1));
    vz = fmaf(L.t[8], n3, fmaf(L.t[5], n2, L.t[2] * n1));
}

// The last steps of every frame search, written once and without contraction of multiply-add pairs, so that every
// kernel that searches frames rounds them alike (their results are compared bit for bit).
#pragma clang fp contract(off)
// unit vector of (x, y, z)
__device__ __forceinline__ void unit_vector(float& x, float& y, float& z) {
    const float inv = 1.0f / sqrtf((x * x + y * y) + z * z);
    x = x * inv; y = y * inv; z = z * inv;
}
// Gram-Schmidt and cross product (models/indexed_lattice_multi_head_attention_cuda.py:475-481; F.normalize eps 1e-12):
// g = normalised part of f2 orthogonal to f1, h = f1 x g
__device__ __forceinline__ void orthonormal_axes(float f1x, float f1y, float f1z, float f2x, float f2y, float f2z,
                                                 float& gx, float& gy, float& gz, float& hx, float& hy, float& hz) {
    const float dot = (f1x * f2x + f1y * f2y) + f1z * f2z;
    gx = f2x - dot * f1x; gy = f2y - dot * f1y; gz = f2z - dot * f1z;
    const float inv = 1.0f / fmaxf(sqrtf((gx * gx + gy * gy) + gz * gz), 1e-12f);
    gx = gx * inv; gy = gy * inv; gz = gz * inv;
    hx = f1y * gz - f1z * gy; hy = f1z * gx - f1x * gz; hz = f1x * gy - f1y * gx;
}
#pragma clang fp contract(fast)

// best candidate of a wavefront: largest score, then lowest pair, then lowest translation
struct Best { float score; int e; int t; };
__device__ __forceinline__ bool better(float s1, int e1, int t1, float s2, int e2, int t2) {
    return s1 > s2 || (s1 == s2 && (e1 < e2 || (e1 == e2 && t1 < t2)));
}
template <int CTRL>
__device__ __forceinline__ void best_dpp(Best& b) {
    const float os = dpp_move<CTRL>(b.score);
    const int oe = __float_as_int(dpp_move<CTRL>(__int_as_float(b.e)));
    const int ot = __float_as_int(dpp_move<CTRL>(__int_as_float(b.t)));
    if (better(os, oe, ot, b.score, b.e, b.t)) { b.score = os; b.e = oe; b.t = ot; }
}
__device__ __forceinline__ void wave_best(Best& b) {
    best_dpp<0xB1>(b); best_dpp<0x4E>(b); best_dpp<0x141>(b); best_dpp<0x140>(b);     // within the rows
    float s0, s1, e0, e1, t0, t1;
    swap32(b.score, s0, s1); swap32(__int_as_float(b.e), e0, e1); swap32(__int_as_float(b.t), t0, t1);
    {
        const bool first = !better(s1, __float_as_int(e1), __float_as_int(t1), s0, __float_as_int(e0), __float_as_int(t0));
        b.score = first ? s0 : s1; b.e = __float_as_int(first ? e0 : e1); b.t = __float_as_int(first ? t0 : t1);
    }
    swap16(b.score, s0, s1); swap16(__int_as_float(b.e), e0, e1); swap16(__int_as_float(b.t), t0, t1);
    {
        const bool first = !better(s1, __float_as_int(e1), __float_as_int(t1), s0, __float_as_int(e0), __float_as_int(t0));
        b.score = first ? s0 : s1; b.e = __float_as_int(first ? e0 : e1); b.t = __float_as_int(first ? t0 : t1);
    }
}

template <int MODE>
__global__ __launch_bounds__(WAVE) void frame_axis_kernel(const KernelArgs P) {
    __shared__ float4 tab[TCAP];
    __shared__ float4 pair_rq[WAVE];        // rpos and q.k of up to 64 pairs
    // one-chunk boxes do not use the table: its memory holds the translation order and per-pair scalars
    uint16_t* const perm = reinterpret_cast<uint16_t*>(tab);              // [TCAP] position -> translation
    float* const reach = reinterpret_cast<float*>(tab) + TCAP / 2;        // [WAVE] see the slab skip below
    float* const phase_of = reach + WAVE;                                 // [WAVE] noise phase of a pair
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

    unsigned long long st_raw = 0;
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
        const Lattice L = item.L;
        const Box bx = item.bx;
        float qi[DH];
#pragma unroll
        for (int c = 0; c < DH; c++) qi[c] = rec_f(rec_cur, REC_QUERY + c);
        const int nchunks = (bx.T + TCAP - 1) / TCAP;
        // One-chunk boxes (T <= TCAP): the lane keeps the shifts of its translations in registers.  The
        // translations with every |n_d| <= 1 (the core, at most 27) come first and are searched two pairs
        // at a time (lanes 0-31 the even pairs of the staged row, lanes 32-63 the odd ones); the others
        // follow in slabs of 64 (both groups in the reference's loop order).  The slabs hold distant
        // translations only: a whole (pair, slab) is skipped when its nearest possible image cannot reach
        // the best score found in the core (smin = smallest shift length of the slab).
        constexpr int SLABS = TCAP / WAVE;
        float cx = 0.f, cy = 0.f, cz = 0.f;
        int ct = 0;
        float sx[SLABS], sy[SLABS], sz[SLABS], smin[SLABS];
        int tt[SLABS];
#pragma unroll
        for (int k = 0; k < SLABS; k++) { sx[k] = sy[k] = sz[k] = 0.0f; smin[k] = 0.0f; tt[k] = 0; }
        int ncore = 0, nout = 0;
        if (nchunks == 1) {
            const float inv_s2 = 1.0f / (float)bx.s2, inv_s3 = 1.0f / (float)bx.s3;
            ncore = min(3, 2 * bx.R1 + 1) * min(3, bx.s2) * min(3, bx.s3);
            nout = bx.T - ncore;
            int seen_core = 0, seen_out = 0;
            wave_sync();                      // the previous item's readers of perm / reach / phase are done
#pragma unroll
            for (int k = 0; k < SLABS; k++)
                if (k * WAVE < bx.T) {
                    const int t = lane + k * WAVE;
                    int n1, n2, n3;
                    box_coords(t, bx, inv_s2, inv_s3, n1, n2, n3);
                    const bool valid = t < bx.T;
                    const bool core = valid && abs(n1) <= 1 && abs(n2) <= 1 && abs(n3) <= 1;
                    const uint64_t mc = __ballot(core), mo = __ballot(valid && !core);
                    if (core) perm[seen_core + lane_prefix(mc)] = (uint16_t)t;
                    else if (valid) perm[ncore + seen_out + lane_prefix(mo)] = (uint16_t)t;
                    seen_core += __popcll(mc);
                    seen_out += __popcll(mo);
                }
            wave_sync();
            auto shift = [&](int t, float& vx, float& vy, float& vz) {
                int n1, n2, n3;
                box_coords(t, bx, inv_s2, inv_s3, n1, n2, n3);
                const float f1 = (float)n1, f2 = (float)n2, f3 = (float)n3;
                vx = fmaf(L.t[6], f3, fmaf(L.t[3], f2, L.t[0] * f1));
                vy = fmaf(L.t[7], f3, fmaf(L.t[4], f2, L.t[1] * f1));
                vz = fmaf(L.t[8], f3, fmaf(L.t[5], f2, L.t[2] * f1));
            };
            ct = perm[min(lane & 31, ncore - 1)];
            shift(ct, cx, cy, cz);
#pragma unroll
            for (int k = 0; k < SLABS; k++)
                if (k * WAVE < nout) {
                    const int pos = ncore + lane + k * WAVE;
                    tt[k] = perm[min(pos, bx.T - 1)];
                    shift(tt[k], sx[k], sy[k], sz[k]);
                    smin[k] = uniform_f(wave_min(pos < bx.T ? sqrtf(fmaf(sx[k], sx[k], fmaf(sy[k], sy[k], sz[k] * sz[k])))
                                                            : 3.0e38f));
                }
        }
        const int e0 = item.e0;
        const int e1 = e0 + item.npairs;

        float f1x = 0.f, f1y = 0.f, f1z = 0.f;     // first axis (input in MODE 1, result otherwise)
        float f2x = 0.f, f2y = 0.f, f2z = 0.f;     // second axis before orthogonalisation
        if (MODE == 1) {
            f1x = uniform_f(P.frame1[((size_t)i * H + h) * 3 + 0]);
            f1y = uniform_f(P.frame1[((size_t)i * H + h) * 3 + 1]);
            f1z = uniform_f(P.frame1[((size_t)i * H + h) * 3 + 2]);
        }

        // pass 0 searches the first axis, pass 1 the second
        for (int pass = (MODE == 1 ? 1 : 0); pass < (MODE == 0 ? 1 : 2); pass++) {
            Best best;
            best.score = -3.0e38f; best.e = 0x7fffffff; best.t = 0x7fffffff;
            for (int eb = e0; eb < e1; eb += WAVE) {
                // stage rpos and q_i.k_j of up to 64 pairs, one per lane (rows of up to 64 pairs keep
                // what the first search staged)
                const bool staged = pass == 1 && MODE == 2 && e1 - e0 <= WAVE;
                wave_sync();
                if (!staged && eb + lane < e1) {
                    const int e = eb + lane;
                    const int64_t j = P.edges[(size_t)P.E + e];
                    const float4* kp = reinterpret_cast<const float4*>(P.k + ((size_t)j * H + h) * DH);
                    float qk = 0.0f;
#pragma unroll
                    for (int c4 = 0; c4 < DH / 4; c4++) {
                        const float4 kv = kp[c4];
                        qk = fmaf(qi[4 * c4 + 0], kv.x, qk);
                        qk = fmaf(qi[4 * c4 + 1], kv.y, qk);
                        qk = fmaf(qi[4 * c4 + 2], kv.z, qk);
                        qk = fmaf(qi[4 * c4 + 3], kv.w, qk);
                    }
                    pair_rq[lane] = make_float4(P.rpos[(size_t)e * 3 + 0], P.rpos[(size_t)e * 3 + 1],
                                                P.rpos[(size_t)e * 3 + 2], qk);
                }
                wave_sync();
                const int ne = min(WAVE, e1 - eb);
                // one candidate: pair e shifted by (vx,vy,vz), translation index t
                // `ordered`: this lane meets its candidates in ascending (pair, translation) order,
                // so the strict comparison alone keeps the first of equal scores
                auto consider = [&](bool ordered, const float4& rq, float phase, int e, int t, float vx, float vy, float vz) {
                    const float dx = rq.x + vx, dy = rq.y + vy, dz = rq.z + vz;
                    const float d2 = fmaf(dx, dx, fmaf(dy, dy, dz * dz));
                    float score = fmaf(a, d2, rq.w);
                    bool ok = d2 > 1e-5f;
                    if (pass == 1) {
                        const float rinv = hw_rsq(d2);
                        const float ac = fabsf((dx * f1x + dy * f1y + dz * f1z) * rinv);
                        score += hw_log2(fmaxf(1.0f - ac, 1e-5f)) * LN2;
                        ok = ok && ac < 0.9999f;
                    }
                    if (noisy) {
                        // uniform in [0,1): golden-ratio sequence over the translations, phase per pair
                        const float un = __builtin_amdgcn_fractf(fmaf((float)t, 0.61803399f, phase));
                        if (pass == 0) score = fmaf(a, d2 + (un - 0.5f) * P.noise, rq.w);
                        else score += (un - 0.5f) * P.noise;
                    }
                    // largest score, then lowest pair, then lowest translation
                    if (ok && (score > best.score ||
                               (!ordered && score == best.score && (e < best.e || (e == best.e && t < best.t))))) {
                        best.score = score; best.e = e; best.t = t;
                    }
                };
                if (nchunks == 1) {
                    if (noisy) {
                        if (lane < ne)
                            phase_of[lane] = hash_uniform(pass ? seed_hi : seed_lo, pass ? seed_lo : seed_hi,
                                                          (uint32_t)((eb + lane) * H + h), (uint32_t)pass);
                        wave_sync();
                    }
                    // the core: one candidate per lane and step, two pairs per step (ascending pairs)
                    {
                        const int half = lane >> 5;
                        const bool core_lane = (lane & 31) < ncore;
#pragma unroll 2
                        for (int m = 0; 2 * m < ne; m++) {
                            const int el = 2 * m + half;
                            const int elc = min(el, ne - 1);
                            const float4 rq = pair_rq[elc];
                            const float ph = noisy ? phase_of[elc] : 0.0f;
                            if (core_lane && el < ne) consider(true, rq, ph, eb + el, ct, cx, cy, cz);
                        }
                    }
                    if (nout > 0) {
                        // A candidate at distance d scores at most q.k + a d^2 + margin (the second search
                        // only subtracts from it; margin = largest noise), and in slab k of pair (i,j)
                        // d >= smin[k] - |r_ij|.  It can matter only if that reaches the best score so far:
                        // smin[k] < reach = |r_ij| + sqrt((best - q.k - margin) / a), widened for rounding.
                        const float glb = -wave_min(-best.score);
                        const float margin = noisy ? (pass == 0 ? fabsf(a) : 1.0f) * 0.5f * P.noise : 0.0f;
                        if (lane < ne) {
                            const float4 rq = pair_rq[lane];
                            const float r = sqrtf(fmaf(rq.x, rq.x, fmaf(rq.y, rq.y, rq.z * rq.z)));
                            const float need = (glb - rq.w - margin) / a;
                            reach[lane] = (a < 0.0f && glb > -1.0e38f)
                                              ? (r + sqrtf(fmaxf(need, 0.0f))) * 1.0001f + 1.0e-3f : 3.0e38f;
                        }
                        wave_sync();
                        const float my_reach = lane < ne ? reach[lane] : -1.0f;
#pragma unroll
                        for (int k = 0; k < SLABS; k++)
                            if (k * WAVE < nout) {
                                uint64_t live = __ballot(smin[k] < my_reach);      // pairs whose slab k is scanned
                                const bool mine = lane + k * WAVE < nout;
                                while (live) {
                                    const int el = __builtin_ctzll(live);
                                    live &= live - 1;
                                    const float4 rq = pair_rq[el];
                                    if (mine) consider(false, rq, noisy ? phase_of[el] : 0.0f, eb + el, tt[k], sx[k], sy[k], sz[k]);
                                }
                            }
                    }
                } else {
                    for (int ch = 0; ch < nchunks; ch++) {
                        const int t0 = ch * TCAP;
                        const int cnt = min(TCAP, bx.T - t0);
                        wave_sync();
                        build_shift_table(tab, t0, cnt, bx, L, lane);
                        wave_sync();
                        for (int el = 0; el < ne; el++) {
                            const float4 rq = pair_rq[el];
                            const int e = eb + el;
                            const float phase = noisy ? hash_uniform(pass ? seed_hi : seed_lo, pass ? seed_lo : seed_hi,
                                                                     (uint32_t)(e * H + h), (uint32_t)pass) : 0.0f;
                            for (int u = lane; u < cnt; u += WAVE) {
                                const float4 v = tab[u];
                                consider(false, rq, phase, e, t0 + u, v.x, v.y, v.z);
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
                const int eb_last = e0 + ((e1 - e0 - 1) / WAVE) * WAVE;      // pairs still staged in LDS
                if (best.e >= eb_last) {
                    const float4 rq = pair_rq[best.e - eb_last];
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
            if (MODE == 0 || MODE == 1) {
                float* o = P.out_frame + ((size_t)i * H + h) * 3;
                if (MODE == 0) { o[0] = f1x; o[1] = f1y; o[2] = f1z; }
                else { o[0] = f2x; o[1] = f2y; o[2] = f2z; }
            } else {
                float gx, gy, gz, hx, hy, hz;
                orthonormal_axes(f1x, f1y, f1z, f2x, f2y, f2z, gx, gy, gz, hx, hy, hz);
                const size_t stride = (size_t)P.N * H * 3;
                float* o = P.out_frame + ((size_t)i * H + h) * 3;
                o[0] = f1x; o[1] = f1y; o[2] = f1z;
                o[stride + 0] = gx; o[stride + 1] = gy; o[stride + 2] = gz;
                o[2 * stride + 0] = hx; o[2 * stride + 1] = hy; o[2 * stride + 2] = hz;
                if (P.frames_to_records) {
                    // the record of this item (already in registers) becomes that of the kernel that
                    // follows: the query makes room for the frames
                    float* r = reinterpret_cast<float*>(P.items + ((size_t)it_cur * H + h) * REC_WORDS + REC_FRAMES);
                    r[0] = f1x; r[1] = f1y; r[2] = f1z;
                    r[3] = gx; r[4] = gy; r[5] = gz;
                    r[6] = hx; r[7] = hy; r[8] = hz;
                }
            }
        }
        st_raw += (unsigned long long)bx.T * (unsigned long long)(e1 - e0);
        it_cur = it_next;
        rec_cur = rec_next;
        it_next = it_cur >= 0 ? queue_redeem(P, h, queue, ticket) : -1;
    }
    if (P.stats && lane == 0) {      // once per wavefront
        if (MODE != 1) atomicAdd(P.stats + STAT_FRAME1_RAW, st_raw);
        if (MODE != 0) atomicAdd(P.stats + STAT_FRAME2_RAW, st_raw);
    }
}

}  // namespace cfh
