/*
 * lattice_oracle.c -- CPU oracle (TEST INFRASTRUCTURE ONLY; never on the product path).
 *
 * A plain-C restatement of the reference's native kernels for the periodic-attention hot path,
 * one scalar loop nest per GPU thread of the reference, same loop order (n1 outermost, n3
 * innermost), same truncation rules and sentinels.  The constants the reference substitutes into
 * the kernel text before NVRTC (models/cuda_funcs/kernel_manager.py:124-149) are run-time fields of
 * orc_params here.  The file is compiled twice, with real = float ("the reference's arithmetic")
 * and real = double ("what the mathematics says"), into one shared library; see oracle/Makefile.
 *
 * Reference text followed, function by function (paths relative to the reference root):
 *   box_ranges ............. models/kernels/real_enc_frame_proj_fwd_length.cu:59-86
 *   orc_pe_fwd ............. models/kernels/real_enc_frame_proj_fwd_length.cu:88-194
 *                            models/kernels/real_enc_frame_proj_fwd_angle.cu:84-209
 *                            models/cuda_funcs/real_space_framed_proj.py:84,105
 *   orc_pe_bwd ............. models/kernels/real_enc_frame_proj_bwd_length.cu:100-237
 *                            models/kernels/real_enc_frame_proj_bwd_angle.cu:104-275
 *                            models/cuda_funcs/real_space_framed_proj.py:183-212
 *   orc_frame1 ............. models/kernels/compute_maximum_frame_each_edge.cu:78-111
 *                            models/cuda_funcs/calc_maximum_frame.py:72-86
 *   orc_frame2 ............. models/kernels/compute_second_frame_each_edge.cu:81-142
 *                            models/cuda_funcs/calc_maximum_frame.py:146-164
 *   orc_dpa_fwd ............ models/kernels/fused_dpa_fwd.cu:46-124
 *   orc_dpa_bwd ............ models/kernels/fused_dpa_bwd.cu:24-126, fused_dpa_bwd_q.cu:13-53
 *   orc_crystal_mean ....... models/kernels/irregular_mean_fwd.cu:13-90 (plain summation order)
 *
 * Deliberate differences from the reference text, all stated where they occur: the tie-breaking
 * noise of the frame search is zero (cuRAND cannot be reproduced), the weight gradients are
 * returned summed over atoms, and "no candidate" outputs are defined (zero vector, -1e30 score).
 *
 * Pinning: checked against the float64 PyTorch oracle (oracle/torch_oracle.py, autograd gradients,
 * no shared formulas) and through it against closed forms; see tests/test_oracle_*.py.  The window
 * index rules, sentinels and range rounding are fixed by the reference text alone.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#ifndef ORC_PARAMS_DEFINED
#define ORC_PARAMS_DEFINED
typedef struct orc_params {
    int32_t H, Dh, K, A;           /* heads, head dim, distance bins, angle bins             */
    int32_t cos_abs;               /* COS_ABS                                                */
    int32_t lattice_range;         /* LATTICE_RANGE                                          */
    int32_t minimum_range;         /* MINIMUM_RANGE                                          */
    int32_t length_range;          /* LENGTH_RANGE = ceil(2*wscale*CUT_SIGMA+1); <=0: full   */
    int32_t angle_range;           /* ANGLE_RANGE                                            */
    int32_t cut_sigma;             /* CUT_SIGMA (4)                                          */
    float dist_max, dist_wscale, angle_sigma;
    float dist_coef, angle_coef;   /* length_rbf_mul, angle_rbf_mul                          */
    float cutoff_radius;
    int32_t grad_coef_quirk;       /* 1: scale the gradients exactly as the reference does   */
} orc_params;
#endif

#define CAT2(a, b) a##b
#define CAT(a, b) CAT2(a, b)
#define FN(name) CAT(name, ORC_SUFFIX)

#if ORC_IS_FLOAT
#define R_SQRT sqrtf
#define R_EXP expf
#define R_LOG logf
#define R_FABS fabsf
#define R_FMIN fminf
#define R_FMAX fmaxf
#else
#define R_SQRT sqrt
#define R_EXP exp
#define R_LOG log
#define R_FABS fabs
#define R_FMIN fmin
#define R_FMAX fmax
#endif

/* Half-widths of the translation box for Gaussian coefficient a.  The arithmetic is float up to the
 * product with the reciprocal length, then double, whatever `real` is: this rule is integer-valued
 * and both builds must agree on it. */
static void FN(box_ranges)(const orc_params* P, float a, const float* rvl, int R[3]) {
    R[0] = R[1] = R[2] = P->lattice_range;
    float cutoff = P->cutoff_radius;
    if (cutoff != 0.0f && rvl) {
        if (cutoff < 0) {
            volatile float s = sqrtf(-0.5f / a);
            volatile float c = s * (-cutoff);
            cutoff = c;
        }
        volatile float c1 = cutoff + 0.01f;
        for (int d = 0; d < 3; d++) {
            volatile float prod = c1 * rvl[d];
            int r = (int)ceil((double)prod / (2.0 * (double)3.141592654f));
            if (P->minimum_range > 0 && r < P->minimum_range) r = P->minimum_range;
            R[d] = r;
        }
    }
}

/* --------------------------------------------------------------------------------------------- */
/* forward: z (E,H), psi (E,H,Dh); optional d2min (E,H) and normalised histograms shat (4,E,H,64) */
void FN(orc_pe_fwd)(const orc_params* P, const ORC_REAL* a_ih, const ORC_REAL* rpos, const ORC_REAL* tvecs,
                    const float* rvlen, const int64_t* batch, const int64_t* edges, int64_t N, int64_t E,
                    const ORC_REAL* W_dist, const ORC_REAL* W_axis, /* (3,H,Dh,A) or NULL */
                    const ORC_REAL* frames,                         /* (3,N,H,3) or NULL  */
                    ORC_REAL* z, ORC_REAL* psi, ORC_REAL* d2min_out) {
    const int H = P->H, Dh = P->Dh, K = P->K, A = P->A;
    const int naxis = (W_axis && frames && A > 0) ? 3 : 0;
#pragma omp parallel for schedule(dynamic, 16)
    for (int64_t tid = 0; tid < E * H; tid++) {
        const int64_t e = tid / H;
        const int h = (int)(tid % H);
        const int64_t i = edges[e];
        const int64_t b = batch[i];
        const ORC_REAL rx = rpos[e * 3], ry = rpos[e * 3 + 1], rz = rpos[e * 3 + 2];
        const ORC_REAL* t = tvecs + b * 9;
        const ORC_REAL a = a_ih[i * H + h];
        int R[3];
        FN(box_ranges)(P, (float)a, rvlen ? rvlen + b * 3 : NULL, R);

        ORC_REAL d2min = (ORC_REAL)1e10;
        for (int n1 = -R[0]; n1 <= R[0]; n1++)
            for (int n2 = -R[1]; n2 <= R[1]; n2++)
                for (int n3 = -R[2]; n3 <= R[2]; n3++) {
                    ORC_REAL dx = rx + t[0] * n1 + t[3] * n2 + t[6] * n3;
                    ORC_REAL dy = ry + t[1] * n1 + t[4] * n2 + t[7] * n3;
                    ORC_REAL dz = rz + t[2] * n1 + t[5] * n2 + t[8] * n3;
                    d2min = R_FMIN(d2min, dx * dx + dy * dy + dz * dz);
                }
        if (d2min_out) d2min_out[tid] = d2min;

        ORC_REAL acc[4][256];
        for (int q = 0; q < 4; q++) memset(acc[q], 0, sizeof(acc[q]));
        ORC_REAL sum = 0;
        for (int n1 = -R[0]; n1 <= R[0]; n1++)
            for (int n2 = -R[1]; n2 <= R[1]; n2++)
                for (int n3 = -R[2]; n3 <= R[2]; n3++) {
                    ORC_REAL dx = rx + t[0] * n1 + t[3] * n2 + t[6] * n3;
                    ORC_REAL dy = ry + t[1] * n1 + t[4] * n2 + t[7] * n3;
                    ORC_REAL dz = rz + t[2] * n1 + t[5] * n2 + t[8] * n3;
                    ORC_REAL d2 = dx * dx + dy * dy + dz * dz;
                    ORC_REAL w = R_EXP(a * (d2 - d2min));
                    sum += w;
                    if (K > 0 && W_dist) {
                        const ORC_REAL step = (ORC_REAL)1.0 / ((ORC_REAL)P->dist_wscale * R_SQRT((ORC_REAL)2.0));
                        const ORC_REAL interval = (ORC_REAL)P->dist_max / K;
                        const ORC_REAL sig = interval * P->dist_wscale;
                        ORC_REAL d = R_SQRT(d2);
                        int start = 0, count = K;
                        if (P->length_range > 0 && K - P->length_range > 8) {
                            start = (int)((d - P->cut_sigma * sig) / interval - 1);   /* C truncation */
                            if (start < 0) start = 0;
                            if (start > K - P->length_range) start = K - P->length_range;
                            count = P->length_range;
                        }
                        ORC_REAL bb = -d / interval * step + step * start;
                        for (int m = 0; m < count; m++) {
                            bb += step;
                            acc[0][m + start] += R_EXP(-bb * bb) * w;
                        }
                    }
                    for (int ax = 0; ax < naxis; ax++) {
                        const ORC_REAL* f = frames + ((ax * N + i) * H + h) * 3;
                        const ORC_REAL as = (ORC_REAL)P->angle_sigma;
                        ORC_REAL step, interval;
                        if (!P->cos_abs) { step = (ORC_REAL)2.0 / ((A - 1) * as * R_SQRT((ORC_REAL)2.0)); interval = (ORC_REAL)2.0 / (A - 1); }
                        else { step = (ORC_REAL)1.0 / ((A - 1) * as * R_SQRT((ORC_REAL)2.0)); interval = (ORC_REAL)1.0 / (A - 1); }
                        const ORC_REAL sigma_inv = (ORC_REAL)1.0 / (as * R_SQRT((ORC_REAL)2.0));
                        ORC_REAL c = (ORC_REAL)1e3;                      /* sentinel: self image */
                        if (d2 > (ORC_REAL)1e-5) c = (dx * f[0] + dy * f[1] + dz * f[2]) / R_SQRT(d2);
                        if (P->cos_abs) c = R_FABS(c);
                        if (P->angle_range > 0 && A - P->angle_range > 8) {
                            ORC_REAL ef = (c + (ORC_REAL)1.0 + P->cut_sigma * as) / interval + (ORC_REAL)1.0;
                            if (ef > (ORC_REAL)A) ef = (ORC_REAL)A;
                            int end = (int)ef;
                            if (end < P->angle_range) end = P->angle_range;
                            ORC_REAL ang = (-c + (ORC_REAL)1.0) * sigma_inv - (A - end) * step;
                            for (int m = 0; m < P->angle_range; m++) {
                                acc[ax + 1][end - m - 1] += R_EXP(-ang * ang) * w;
                                ang -= step;
                            }
                        } else {
                            ORC_REAL ang = (-c + (ORC_REAL)1.0) * sigma_inv - (A - 1) * step;
                            for (int m = 0; m < A; m++) {
                                acc[ax + 1][m] += R_EXP(-ang * ang) * w;
                                ang += step;
                            }
                        }
                    }
                }
        if (K > 0 && W_dist && psi) {
            for (int c = 0; c < Dh; c++) {
                ORC_REAL sv = 0;
                const ORC_REAL* W = W_dist + ((int64_t)h * Dh + c) * K;
                for (int k = 0; k < K; k++) sv += W[k] * acc[0][k];
                ORC_REAL out = sv / sum * P->dist_coef;
                for (int ax = 0; ax < naxis; ax++) {
                    ORC_REAL sa = 0;
                    const ORC_REAL* Wa = W_axis + (((int64_t)ax * H + h) * Dh + c) * A;
                    for (int m = 0; m < A; m++) sa += Wa[m] * acc[ax + 1][m];
                    out += sa / sum * P->angle_coef;
                }
                psi[tid * Dh + c] = out;
            }
        }
        z[tid] = R_LOG(sum) + d2min * a;
    }
}

/* --------------------------------------------------------------------------------------------- */
/* backward: ga (N,H), gW_dist (H,Dh,K), gW_axis (3,H,Dh,A) -- the weight gradients summed over the
 * per-atom partials the reference leaves to autograd's broadcast reduction.                      */
void FN(orc_pe_bwd)(const orc_params* P, const ORC_REAL* a_ih, const ORC_REAL* rpos, const ORC_REAL* tvecs,
                    const float* rvlen, const int64_t* batch, const int64_t* e_start, int64_t N, int64_t E,
                    const ORC_REAL* W_dist, const ORC_REAL* W_axis, const ORC_REAL* frames,
                    const ORC_REAL* z, const ORC_REAL* gz, const ORC_REAL* gpsi, ORC_REAL* ga,
                    ORC_REAL* gW_dist, ORC_REAL* gW_axis) {
    const int H = P->H, Dh = P->Dh, K = P->K, A = P->A;
    const int naxis = (W_axis && frames && A > 0) ? 3 : 0;
    const int has_len = (K > 0 && W_dist);
    const int64_t wl = (int64_t)H * Dh * K, wa = (int64_t)3 * H * Dh * A;
    /* per-atom partials, as the reference allocates them (gW_k of shape (N,H,Dh,K)) */
    ORC_REAL* part_l = has_len ? (ORC_REAL*)calloc((size_t)(N * Dh * K * H), sizeof(ORC_REAL)) : NULL;
    ORC_REAL* part_a = naxis ? (ORC_REAL*)calloc((size_t)(N * 3 * Dh * A * H), sizeof(ORC_REAL)) : NULL;
#pragma omp parallel for schedule(dynamic, 4)
    for (int64_t tid = 0; tid < N * H; tid++) {
        const int64_t i = tid / H;
        const int h = (int)(tid % H);
        const int64_t b = batch[i];
        const ORC_REAL* t = tvecs + b * 9;
        const ORC_REAL a = a_ih[i * H + h];
        int R[3];
        FN(box_ranges)(P, (float)a, rvlen ? rvlen + b * 3 : NULL, R);
        ORC_REAL ga_z = 0, ga_len = 0, ga_ang = 0;
        for (int64_t e = e_start[i]; e < e_start[i + 1]; e++) {
            const ORC_REAL rx = rpos[e * 3], ry = rpos[e * 3 + 1], rz = rpos[e * 3 + 2];
            const ORC_REAL ze = z[e * H + h];
            const ORC_REAL* gv = gpsi ? gpsi + (e * H + h) * Dh : NULL;
            for (int enc = 0; enc < 1 + naxis; enc++) {
                if (enc == 0 && !has_len) continue;
                const int D = enc == 0 ? K : A;
                const ORC_REAL* W = enc == 0 ? W_dist + (int64_t)h * Dh * K
                                             : W_axis + (((int64_t)(enc - 1) * H + h) * Dh) * A;
                ORC_REAL G[256], sv[256];
                for (int k = 0; k < D; k++) { G[k] = 0; sv[k] = 0; }
                for (int c = 0; c < Dh; c++)
                    for (int k = 0; k < D; k++) G[k] += W[c * D + k] * gv[c];
                const ORC_REAL* f = enc > 0 ? frames + (((enc - 1) * N + i) * H + h) * 3 : NULL;
                ORC_REAL px_avr = 0, pbg_avr = 0, cov = 0;
                for (int n1 = -R[0]; n1 <= R[0]; n1++)
                    for (int n2 = -R[1]; n2 <= R[1]; n2++)
                        for (int n3 = -R[2]; n3 <= R[2]; n3++) {
                            ORC_REAL dx = rx + t[0] * n1 + t[3] * n2 + t[6] * n3;
                            ORC_REAL dy = ry + t[1] * n1 + t[4] * n2 + t[7] * n3;
                            ORC_REAL dz = rz + t[2] * n1 + t[5] * n2 + t[8] * n3;
                            ORC_REAL d2 = dx * dx + dy * dy + dz * dz;
                            ORC_REAL p = R_EXP(a * d2 - ze);
                            ORC_REAL px = d2 * p;
                            ORC_REAL d = R_SQRT(d2);
                            px_avr += px;
                            ORC_REAL bg = 0;
                            if (enc == 0) {
                                const ORC_REAL step = (ORC_REAL)1.0 / ((ORC_REAL)P->dist_wscale * R_SQRT((ORC_REAL)2.0));
                                const ORC_REAL interval = (ORC_REAL)P->dist_max / K;
                                const ORC_REAL sig = interval * P->dist_wscale;
                                int start = 0, count = K;
                                if (P->length_range > 0 && K - P->length_range > 8) {
                                    start = (int)((d - P->cut_sigma * sig) / interval - 1);
                                    if (start > K - P->length_range) start = K - P->length_range;
                                    if (start < 0) start = 0;
                                    count = P->length_range;
                                }
                                ORC_REAL bb = -d / interval * step + step * start;
                                for (int m = 0; m < count; m++) {
                                    bb += step;
                                    ORC_REAL g = R_EXP(-bb * bb);
                                    bg += g * G[start + m];
                                    sv[start + m] += g * p;
                                }
                            } else {
                                const ORC_REAL as = (ORC_REAL)P->angle_sigma;
                                ORC_REAL step, interval;
                                if (!P->cos_abs) { step = (ORC_REAL)2.0 / ((A - (ORC_REAL)1.0) * as * R_SQRT((ORC_REAL)2.0)); interval = (ORC_REAL)2.0 / (A - (ORC_REAL)1.0); }
                                else { step = (ORC_REAL)1.0 / ((A - (ORC_REAL)1.0) * as * R_SQRT((ORC_REAL)2.0)); interval = (ORC_REAL)1.0 / (A - (ORC_REAL)1.0); }
                                const ORC_REAL sigma_inv = (ORC_REAL)1.0 / (as * R_SQRT((ORC_REAL)2.0));
                                ORC_REAL c = (ORC_REAL)1e3;
                                if (d2 > (ORC_REAL)1e-5) c = (dx * f[0] + dy * f[1] + dz * f[2]) / d;
                                if (P->cos_abs) c = R_FABS(c);
                                if (P->angle_range > 0 && A - P->angle_range > 8) {
                                    ORC_REAL ef = (c + (ORC_REAL)1.0 + P->cut_sigma * as) / interval + 1;
                                    if (ef > (ORC_REAL)A) ef = (ORC_REAL)A;
                                    int end = (int)ef;
                                    if (end < P->angle_range) end = P->angle_range;
                                    ORC_REAL ang = (-c + (ORC_REAL)1.0) * sigma_inv - (A - end) * step;
                                    for (int m = 0; m < P->angle_range; m++) {
                                        ORC_REAL g = R_EXP(-ang * ang);
                                        sv[end - 1 - m] += g * p;
                                        bg += g * G[end - 1 - m];
                                        ang -= step;
                                    }
                                } else {
                                    ORC_REAL ang = (-c + (ORC_REAL)1.0) * sigma_inv - (A - 1) * step;
                                    for (int m = 0; m < A; m++) {
                                        ORC_REAL g = R_EXP(-ang * ang);
                                        sv[m] += g * p;
                                        bg += g * G[m];
                                        ang += step;
                                    }
                                }
                            }
                            cov += px * bg;
                            pbg_avr += p * bg;
                        }
                cov -= px_avr * pbg_avr;
                if (enc == 0) { ga_z += px_avr * gz[e * H + h]; ga_len += cov; }
                else ga_ang += cov;
                ORC_REAL* dst = enc == 0 ? part_l + (i * H + h) * Dh * K
                                         : part_a + (((enc - 1) * N + i) * H + h) * Dh * A;
                for (int c = 0; c < Dh; c++)
                    for (int k = 0; k < D; k++) dst[c * D + k] += sv[k] * gv[c];
            }
            if (!has_len) {      /* z only: the length kernel still runs and yields gz * sum p d^2 */
                ORC_REAL px_avr = 0;
                for (int n1 = -R[0]; n1 <= R[0]; n1++)
                    for (int n2 = -R[1]; n2 <= R[1]; n2++)
                        for (int n3 = -R[2]; n3 <= R[2]; n3++) {
                            ORC_REAL dx = rx + t[0] * n1 + t[3] * n2 + t[6] * n3;
                            ORC_REAL dy = ry + t[1] * n1 + t[4] * n2 + t[7] * n3;
                            ORC_REAL dz = rz + t[2] * n1 + t[5] * n2 + t[8] * n3;
                            ORC_REAL d2 = dx * dx + dy * dy + dz * dz;
                            px_avr += d2 * R_EXP(a * d2 - ze);
                        }
                ga_z += px_avr * gz[e * H + h];
            }
        }
        /* real_space_framed_proj.py:183,209: ga = c_d*(gz part + cov_len) + c_a*sum_axis cov.  The exact
         * gradient scales only the covariance terms. */
        if (P->grad_coef_quirk) ga[tid] = P->dist_coef * (ga_z + ga_len) + P->angle_coef * ga_ang;
        else ga[tid] = ga_z + P->dist_coef * ga_len + P->angle_coef * ga_ang;
    }
    /* reduction over atoms (done by autograd's sum_to_size in the reference) and the coefficient of
     * real_space_framed_proj.py:210-212 (gW_axis *= c_a; gW_dist unscaled in the reference). */
    if (has_len && gW_dist) {
        const ORC_REAL sc = P->grad_coef_quirk ? (ORC_REAL)1.0 : (ORC_REAL)P->dist_coef;
        for (int64_t x = 0; x < wl; x++) gW_dist[x] = 0;
        for (int64_t i = 0; i < N; i++)
            for (int64_t x = 0; x < wl; x++) gW_dist[x] += part_l[i * wl + x] * sc;
    }
    if (naxis && gW_axis) {
        const int64_t per = (int64_t)H * Dh * A;
        for (int64_t x = 0; x < wa; x++) gW_axis[x] = 0;
        for (int ax = 0; ax < 3; ax++)
            for (int64_t i = 0; i < N; i++)
                for (int64_t x = 0; x < per; x++)
                    gW_axis[ax * per + x] += part_a[(ax * N + i) * per + x] * (ORC_REAL)P->angle_coef;
    }
    free(part_l);
    free(part_a);
}

/* --------------------------------------------------------------------------------------------- */
/* frames.  q must be pre-divided by sqrt(Dh).  Zero noise: the strict comparisons keep the first
 * image in loop order; across edges the lowest edge index wins (plain arg-max).                   */
void FN(orc_frame1)(const orc_params* P, const ORC_REAL* q, const ORC_REAL* k, const ORC_REAL* a_ih,
                    const ORC_REAL* rpos, const ORC_REAL* tvecs, const float* rvlen, const int64_t* batch,
                    const int64_t* edges, int64_t N, int64_t E, ORC_REAL* frame1) {
    const int H = P->H, Dh = P->Dh;
    ORC_REAL* dir = (ORC_REAL*)malloc(sizeof(ORC_REAL) * (size_t)(E * H * 3));
    ORC_REAL* val = (ORC_REAL*)malloc(sizeof(ORC_REAL) * (size_t)(E * H));
#pragma omp parallel for schedule(dynamic, 16)
    for (int64_t tid = 0; tid < E * H; tid++) {
        const int64_t e = tid / H;
        const int h = (int)(tid % H);
        const int64_t i = edges[e], j = edges[E + e];
        const int64_t b = batch[i];
        const ORC_REAL rx = rpos[e * 3], ry = rpos[e * 3 + 1], rz = rpos[e * 3 + 2];
        const ORC_REAL* t = tvecs + b * 9;
        const ORC_REAL a = a_ih[i * H + h];
        int R[3];
        FN(box_ranges)(P, (float)a, rvlen ? rvlen + b * 3 : NULL, R);
        ORC_REAL d2_min = (ORC_REAL)1e10, vx = 0, vy = 0, vz = 0;
        for (int n1 = -R[0]; n1 <= R[0]; n1++)
            for (int n2 = -R[1]; n2 <= R[1]; n2++)
                for (int n3 = -R[2]; n3 <= R[2]; n3++) {
                    ORC_REAL dx = rx + t[0] * n1 + t[3] * n2 + t[6] * n3;
                    ORC_REAL dy = ry + t[1] * n1 + t[4] * n2 + t[7] * n3;
                    ORC_REAL dz = rz + t[2] * n1 + t[5] * n2 + t[8] * n3;
                    ORC_REAL d2 = dx * dx + dy * dy + dz * dz;
                    ORC_REAL d = R_SQRT(d2);
                    if (d2 > (ORC_REAL)1e-5 && d2_min > d2) {
                        d2_min = d2;
                        vx = dx / d; vy = dy / d; vz = dz / d;
                    }
                }
        ORC_REAL qk = 0;
        for (int c = 0; c < Dh; c++) qk += q[(i * H + h) * Dh + c] * k[(j * H + h) * Dh + c];
        dir[tid * 3] = vx; dir[tid * 3 + 1] = vy; dir[tid * 3 + 2] = vz;
        val[tid] = qk + a * d2_min;
    }
    for (int64_t x = 0; x < N * H * 3; x++) frame1[x] = 0;
    ORC_REAL* best = (ORC_REAL*)malloc(sizeof(ORC_REAL) * (size_t)(N * H));
    for (int64_t x = 0; x < N * H; x++) best[x] = (ORC_REAL)-1e10;
    for (int64_t e = 0; e < E; e++)
        for (int h = 0; h < H; h++) {
            const int64_t i = edges[e];
            if (val[e * H + h] > best[i * H + h]) {
                best[i * H + h] = val[e * H + h];
                for (int d = 0; d < 3; d++) frame1[(i * H + h) * 3 + d] = dir[(e * H + h) * 3 + d];
            }
        }
    free(dir); free(val); free(best);
}

void FN(orc_frame2)(const orc_params* P, const ORC_REAL* q, const ORC_REAL* k, const ORC_REAL* a_ih,
                    const ORC_REAL* rpos, const ORC_REAL* tvecs, const float* rvlen, const int64_t* batch,
                    const int64_t* edges, const ORC_REAL* frame1, int64_t N, int64_t E, ORC_REAL* frame2) {
    const int H = P->H, Dh = P->Dh;
    ORC_REAL* dir = (ORC_REAL*)calloc((size_t)(E * H * 3), sizeof(ORC_REAL));
    ORC_REAL* val = (ORC_REAL*)malloc(sizeof(ORC_REAL) * (size_t)(E * H));
#pragma omp parallel for schedule(dynamic, 16)
    for (int64_t tid = 0; tid < E * H; tid++) {
        const int64_t e = tid / H;
        const int h = (int)(tid % H);
        const int64_t i = edges[e], j = edges[E + e];
        const int64_t b = batch[i];
        const ORC_REAL rx = rpos[e * 3], ry = rpos[e * 3 + 1], rz = rpos[e * 3 + 2];
        const ORC_REAL* t = tvecs + b * 9;
        const ORC_REAL a = a_ih[i * H + h];
        int R[3];
        FN(box_ranges)(P, (float)a, rvlen ? rvlen + b * 3 : NULL, R);
        ORC_REAL d2min = (ORC_REAL)1e10;
        for (int n1 = -R[0]; n1 <= R[0]; n1++)
            for (int n2 = -R[1]; n2 <= R[1]; n2++)
                for (int n3 = -R[2]; n3 <= R[2]; n3++) {
                    ORC_REAL dx = rx + t[0] * n1 + t[3] * n2 + t[6] * n3;
                    ORC_REAL dy = ry + t[1] * n1 + t[4] * n2 + t[7] * n3;
                    ORC_REAL dz = rz + t[2] * n1 + t[5] * n2 + t[8] * n3;
                    ORC_REAL d2 = dx * dx + dy * dy + dz * dz;
                    if (d2 > (ORC_REAL)1e-5) d2min = R_FMIN(d2min, d2);
                }
        const ORC_REAL f1x = frame1[(i * H + h) * 3], f1y = frame1[(i * H + h) * 3 + 1], f1z = frame1[(i * H + h) * 3 + 2];
        ORC_REAL max_val = (ORC_REAL)-1e15, second_value = (ORC_REAL)-1e30, sx = 0, sy = 0, sz = 0;
        for (int n1 = -R[0]; n1 <= R[0]; n1++)
            for (int n2 = -R[1]; n2 <= R[1]; n2++)
                for (int n3 = -R[2]; n3 <= R[2]; n3++) {
                    ORC_REAL dx = rx + t[0] * n1 + t[3] * n2 + t[6] * n3;
                    ORC_REAL dy = ry + t[1] * n1 + t[4] * n2 + t[7] * n3;
                    ORC_REAL dz = rz + t[2] * n1 + t[5] * n2 + t[8] * n3;
                    ORC_REAL d2 = dx * dx + dy * dy + dz * dz;
                    ORC_REAL d = R_SQRT(d2);
                    if (d2 > (ORC_REAL)1e-5) {
                        ORC_REAL ux = dx / d, uy = dy / d, uz = dz / d;
                        ORC_REAL ct = ux * f1x + uy * f1y + uz * f1z;
                        ORC_REAL v = a * (d2 - d2min) + R_LOG(R_FMAX((ORC_REAL)1.0 - R_FABS(ct), (ORC_REAL)1e-5));
                        if (v > max_val && R_FABS(ct) < (ORC_REAL)0.9999) {
                            max_val = v;
                            sx = ux; sy = uy; sz = uz;
                            second_value = v + a * d2min;
                        }
                    }
                }
        ORC_REAL qk = 0;
        for (int c = 0; c < Dh; c++) qk += q[(i * H + h) * Dh + c] * k[(j * H + h) * Dh + c];
        dir[tid * 3] = sx; dir[tid * 3 + 1] = sy; dir[tid * 3 + 2] = sz;
        val[tid] = qk + second_value;
    }
    for (int64_t x = 0; x < N * H * 3; x++) frame2[x] = 0;
    ORC_REAL* best = (ORC_REAL*)malloc(sizeof(ORC_REAL) * (size_t)(N * H));
    for (int64_t x = 0; x < N * H; x++) best[x] = (ORC_REAL)-1e10;
    for (int64_t e = 0; e < E; e++)
        for (int h = 0; h < H; h++) {
            const int64_t i = edges[e];
            if (val[e * H + h] > best[i * H + h]) {
                best[i * H + h] = val[e * H + h];
                for (int d = 0; d < 3; d++) frame2[(i * H + h) * 3 + d] = dir[(e * H + h) * 3 + d];
            }
        }
    free(dir); free(val); free(best);
}

/* --------------------------------------------------------------------------------------------- */
/* softmax over neighbours: out (N,H,Dh), prob (E,H).  q pre-divided by sqrt(Dh).                */
void FN(orc_dpa_fwd)(int H, int Dh, const ORC_REAL* q, const ORC_REAL* k, const ORC_REAL* v,
                     const ORC_REAL* z, const ORC_REAL* psi, const int64_t* edges,
                     const int64_t* e_start, int64_t N, int64_t E, ORC_REAL* prob, ORC_REAL* out) {
#pragma omp parallel for schedule(dynamic, 16)
    for (int64_t tid = 0; tid < N * H; tid++) {
        const int64_t i = tid / H;
        const int h = (int)(tid % H);
        ORC_REAL mx = (ORC_REAL)-1e20;
        for (int64_t e = e_start[i]; e < e_start[i + 1]; e++) {
            const int64_t j = edges[E + e];
            ORC_REAL at = 0;
            for (int c = 0; c < Dh; c++) at += q[tid * Dh + c] * k[(j * H + h) * Dh + c];
            if (z) at += z[e * H + h];
            prob[e * H + h] = at;
            mx = R_FMAX(mx, at);
        }
        ORC_REAL sum = 0;
        for (int64_t e = e_start[i]; e < e_start[i + 1]; e++) {
            ORC_REAL w = R_EXP(prob[e * H + h] - mx);
            prob[e * H + h] = w;
            sum += w;
        }
        for (int c = 0; c < Dh; c++) out[tid * Dh + c] = 0;
        for (int64_t e = e_start[i]; e < e_start[i + 1]; e++) {
            const int64_t j = edges[E + e];
            prob[e * H + h] /= sum;
            for (int c = 0; c < Dh; c++) {
                ORC_REAL val = v[(j * H + h) * Dh + c];
                if (psi) val += psi[(e * H + h) * Dh + c];
                out[tid * Dh + c] += val * prob[e * H + h];
            }
        }
    }
}

/* gradients of the above: gq, gk, gv (N,H,Dh), gz (E,H), gpsi (E,H,Dh) */
void FN(orc_dpa_bwd)(int H, int Dh, const ORC_REAL* q, const ORC_REAL* k, const ORC_REAL* v,
                     const ORC_REAL* psi, const int64_t* edges, const int64_t* e_start, int64_t N,
                     int64_t E, const ORC_REAL* prob, const ORC_REAL* out, const ORC_REAL* gout,
                     ORC_REAL* gq, ORC_REAL* gk, ORC_REAL* gv, ORC_REAL* gz, ORC_REAL* gpsi) {
    for (int64_t x = 0; x < N * H * Dh; x++) { gq[x] = 0; gk[x] = 0; gv[x] = 0; }
    for (int64_t i = 0; i < N; i++)
        for (int h = 0; h < H; h++)
            for (int64_t e = e_start[i]; e < e_start[i + 1]; e++) {
                const int64_t j = edges[E + e];
                const ORC_REAL p = prob[e * H + h];
                ORC_REAL gs = 0;
                for (int c = 0; c < Dh; c++) {
                    const ORC_REAL tt = gout[(i * H + h) * Dh + c] * p;
                    gv[(j * H + h) * Dh + c] += tt;
                    ORC_REAL val = v[(j * H + h) * Dh + c];
                    if (psi) { val += psi[(e * H + h) * Dh + c]; gpsi[(e * H + h) * Dh + c] = tt; }
                    gs += (val - out[(i * H + h) * Dh + c]) * tt;
                }
                gz[e * H + h] = gs;
                for (int c = 0; c < Dh; c++) {
                    gk[(j * H + h) * Dh + c] += gs * q[(i * H + h) * Dh + c];
                    gq[(i * H + h) * Dh + c] += gs * k[(j * H + h) * Dh + c];
                }
            }
}

/* per-crystal mean of x (N,D) -> (B,D); start (B+1) */
void FN(orc_crystal_mean)(const ORC_REAL* x, const int64_t* start, int64_t B, int64_t D, ORC_REAL* out) {
    for (int64_t b = 0; b < B; b++)
        for (int64_t c = 0; c < D; c++) {
            ORC_REAL s = 0;
            for (int64_t n = start[b]; n < start[b + 1]; n++) s += x[n * D + c];
            out[b * D + c] = s / (ORC_REAL)(start[b + 1] - start[b]);
        }
}

#undef R_SQRT
#undef R_EXP
#undef R_LOG
#undef R_FABS
#undef R_FMIN
#undef R_FMAX
