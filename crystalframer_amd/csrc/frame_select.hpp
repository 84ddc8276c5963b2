// Dynamic "max" frame selection.  For every (atom i, head h) the first axis points to the most
// attended periodic image, the second (before orthogonalisation) to the image maximising the
// attention logit plus log(1-|cos|) to the first axis.  One wavefront scans all neighbours j and
// all translations n of an (i,h) item and keeps the joint arg-max, which replaces the reference's
// per-edge kernel + gathered q.k product + third-party segmented arg-max
// (models/kernels/compute_maximum_frame_each_edge.cu:78-111,
//  models/kernels/compute_second_frame_each_edge.cu:81-142,
//  models/cuda_funcs/calc_maximum_frame.py:72-86,146-164).
//
// Tie rule with zero noise: per pair the first image in the reference's loop order wins (its
// strict comparisons), across pairs the lowest edge index wins.  With noise > 0 every candidate's
// key is perturbed by a counter-based uniform in (-noise/2, noise/2) (the reference draws from
// cuRAND XORWOW seeded by numpy; its stream cannot be reproduced).
#pragma once
#include "device_common.hpp"

namespace cfh {

__device__ __forceinline__ void shift_of(int t, const Box& bx, const Lattice& L, float& vx, float& vy,
                                         float& vz) {
    const int i3 = t % bx.s3;
    const int q = t / bx.s3;
    const int i2 = q % bx.s2;
    const int i1 = q / bx.s2;
    const float n1 = (float)(i1 - bx.R1), n2 = (float)(i2 - bx.R2), n3 = (float)(i3 - bx.R3);
    vx = fmaf(L.t[6], n3, fmaf(L.t[3], n2, L.t[0] * n1));
    vy = fmaf(L.t[7], n3, fmaf(L.t[4], n2, L.t[1] * n1));
    vz = fmaf(L.t[8], n3, fmaf(L.t[5], n2, L.t[2] * n1));
}

template <bool SECOND>
__global__ __launch_bounds__(WAVE) void frame_axis_kernel(const KernelArgs P) {
    __shared__ float4 tab[TCAP];
    const int lane = threadIdx.x;
    const int H = P.H;
    const int h = blockIdx.x % H;
    const bool noisy = P.noise > 0.0f;

    for (;;) {
        const int it = next_item(P.counters + h, lane);
        if (it >= P.N) break;
        const int i = P.order ? uniform_i(P.order[it]) : it;
        const int b = uniform_i((int)P.batch[i]);
        const float a = uniform_f(P.a_ih[(size_t)i * H + h]);
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
        float qi[DH];
#pragma unroll
        for (int c = 0; c < DH; c++) qi[c] = uniform_f(P.q[((size_t)i * H + h) * DH + c]);
        float f1x = 0.f, f1y = 0.f, f1z = 0.f;
        if (SECOND) {
            f1x = uniform_f(P.frame1[((size_t)i * H + h) * 3 + 0]);
            f1y = uniform_f(P.frame1[((size_t)i * H + h) * 3 + 1]);
            f1z = uniform_f(P.frame1[((size_t)i * H + h) * 3 + 2]);
        }
        const int nchunks = (bx.T + TCAP - 1) / TCAP;
        if (nchunks == 1) {
            __syncthreads();
            build_shift_table(tab, 0, bx.T, bx, L, lane);
            __syncthreads();
        }
        const int e0 = uniform_i((int)P.e_start[i]);
        const int e1 = uniform_i((int)P.e_start[i + 1]);

        float best_score = -3.0e38f;
        float bx_ = 0.f, by_ = 0.f, bz_ = 0.f;      // best direction (unnormalised image vector)

        for (int eb = e0; eb < e1; eb += WAVE) {
            // q_i . k_j for up to 64 neighbours, one per lane
            float qk_lane = 0.0f;
            if (eb + lane < e1) {
                const int64_t j = P.edges[(size_t)P.E + eb + lane];
                const float4* kp = reinterpret_cast<const float4*>(P.k + ((size_t)j * H + h) * DH);
#pragma unroll
                for (int c4 = 0; c4 < DH / 4; c4++) {
                    const float4 kv = kp[c4];
                    qk_lane = fmaf(qi[4 * c4 + 0], kv.x, qk_lane);
                    qk_lane = fmaf(qi[4 * c4 + 1], kv.y, qk_lane);
                    qk_lane = fmaf(qi[4 * c4 + 2], kv.z, qk_lane);
                    qk_lane = fmaf(qi[4 * c4 + 3], kv.w, qk_lane);
                }
            }
            const int ne = min(WAVE, e1 - eb);
            for (int el = 0; el < ne; el++) {
                const int e = eb + el;
                const float qk = __shfl(qk_lane, el, WAVE);
                const float rx = uniform_f(P.rpos[(size_t)e * 3 + 0]);
                const float ry = uniform_f(P.rpos[(size_t)e * 3 + 1]);
                const float rz = uniform_f(P.rpos[(size_t)e * 3 + 2]);

                // ---- nearest image with d^2 > 1e-5 (first in loop order on ties)
                float bd = 3.0e38f;
                int bt = 0x7fffffff;
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
                        const float d2 = fmaf(dx, dx, fmaf(dy, dy, dz * dz));
                        float key = d2;
                        if (noisy && !SECOND)
                            key += (hash_uniform(P.seed_lo, P.seed_hi, (uint32_t)(e * H + h), (uint32_t)(t0 + u)) - 0.5f) * P.noise;
                        if (d2 > 1e-5f && key < bd) { bd = key; bt = t0 + u; }
                    }
                }
                wave_argmin(bd, bt);
                if (bt == 0x7fffffff) continue;      // no image at all: cannot happen for R >= 1

                if (!SECOND) {
                    const float score = qk + a * bd;
                    if (score > best_score) {
                        best_score = score;
                        float vx, vy, vz;
                        shift_of(bt, bx, L, vx, vy, vz);
                        bx_ = rx + vx; by_ = ry + vy; bz_ = rz + vz;
                    }
                } else {
                    const float d2min = bd;
                    float bv = -3.0e38f;
                    int bt2 = 0x7fffffff;
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
                            const float d2 = fmaf(dx, dx, fmaf(dy, dy, dz * dz));
                            if (d2 > 1e-5f) {
                                const float rinv = hw_rsq(d2);
                                const float ac = fabsf((dx * f1x + dy * f1y + dz * f1z) * rinv);
                                float val = a * (d2 - d2min) + hw_log2(fmaxf(1.0f - ac, 1e-5f)) * LN2;
                                if (noisy)
                                    val += (hash_uniform(P.seed_lo, P.seed_hi, (uint32_t)(e * H + h), (uint32_t)(t0 + u)) - 0.5f) * P.noise;
                                if (ac < 0.9999f && val > bv) { bv = val; bt2 = t0 + u; }
                            }
                        }
                    }
                    wave_argmax(bv, bt2);
                    if (bt2 == 0x7fffffff) continue;  // every image collinear with the first axis
                    const float score = qk + (bv + a * d2min);
                    if (score > best_score) {
                        best_score = score;
                        float vx, vy, vz;
                        shift_of(bt2, bx, L, vx, vy, vz);
                        bx_ = rx + vx; by_ = ry + vy; bz_ = rz + vz;
                    }
                }
            }
        }
        if (lane == 0) {
            const float d2 = bx_ * bx_ + by_ * by_ + bz_ * bz_;
            const float inv = d2 > 0.0f ? 1.0f / sqrtf(d2) : 0.0f;
            float* o = P.out_frame + ((size_t)i * H + h) * 3;
            o[0] = bx_ * inv; o[1] = by_ * inv; o[2] = bz_ * inv;
            if (P.stats)
                atomicAdd(P.stats + (SECOND ? STAT_FRAME2_RAW : STAT_FRAME1_RAW),
                          (unsigned long long)bx.T * (unsigned long long)(e1 - e0));
        }
    }
}

}  // namespace cfh
