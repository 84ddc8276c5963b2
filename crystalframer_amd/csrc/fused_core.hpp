// Fused attention core: lattice sums, softmax over the pairs of an atom and the value encoding in ONE pass per
// (atom i, head h), with ONE histogram per (atom, head) instead of one per (pair, head).
//
// The attention output is linear in the value encoding,
//     out_i = sum_j P_ij (v_j + psi_ij),   psi_ij = W . shat_ij,   shat_ij = sum_n p_n b(image n of pair ij),
// so  sum_j P_ij psi_ij = W . T_i  with  T_i = sum_j sum_n P_ij p_n b(.): the per-image basis values can be
// scattered, weighted by P_ij p_n, into one histogram per item, and the projection W is applied once per item by
// a small MFMA product afterwards.  psi (E,H,16) and the per-pair histograms never exist.  The softmax weights
// P_ij are not known before all pairs of the row have been seen, so the pass keeps a running maximum of the
// logits (q_i.k_j + z_ij) and rescales histogram, value accumulator and denominator when it grows (online
// softmax).  What the reference computes in five kernels and a tensor sum
// (models/kernels/real_enc_frame_proj_fwd_length.cu, ..._fwd_angle.cu, fused_dpa_fwd.cu;
//  models/cuda_funcs/real_space_framed_proj.py:21-120, fused_dpa.py:17-63) is one kernel plus the projection here.
//
// Two further changes of formulation (same mathematics, different arithmetic):
//   * sorted translations.  For the usual box (half-width 2 = 125 translations) a table of the box's shifts
//     sorted by length is made once per crystal.  An image at shift s of a pair at r lies at distance
//     >= |s| - |r|, so the nearest image of a pair is found in the prefix |s| <= 2|r| and every image whose
//     weight can reach 2^-skip of the heaviest one in the prefix |s| <= |r| + sqrt(d2min + skip/(-a log2 e)):
//     the two light sweeps read a fraction of the box instead of all of it twice.
//   * angle encoding by local moments.  The Gaussian basis of the cosine has sigma = wscale bins (4), so around
//     the bin m* nearest to x the value of every basis function is a short power series in the offset
//     eps = 2 (u - m*) in [-1,1] (u = x in bin units):
//         exp(-((m - u)/ws)^2 / 2) = sum_o eps^o D_o(m - m*),  D_o(d) = exp(-(d/ws)^2/2) He_o(d/ws) / (o! (2 ws)^o)
//     (generating function of the Hermite polynomials; truncated after NORD = 5 terms the error is below 2e-6 of
//     the peak, 6 terms: 1e-7).  A term therefore adds NORD moments w eps^o at ONE bin per axis instead of a 33-bin window, and
//     the constant matrices D_o are folded into the projection weights (core_wcat_kernel).  This is the FULL
//     basis (no +-4 sigma truncation), i.e. the pure-PyTorch formulation of the reference
//     (models/indexed_lattice_multi_head_attention.py:580-588) rather than the windowed one of its CUDA kernels.
//     The distance basis (sigma = 1 bin) keeps its truncated window.
//
// Histogram of an item ("hist", HW words): [0,64) distance bins, then for axis ax and order o the 64 moment bins
// at 64 + (ax NORD + o) 64.  It is accumulated in LDS as signed 32-bit fixed point (round to nearest) in units of
// 2^30 / npairs relative to the heaviest pair of the row so far, and written out normalised as float32.
#pragma once
#include <type_traits>
#include "device_common.hpp"

namespace cfh {

constexpr int FC_TCAP = 128;                    // translations per table chunk (the sorted table of the usual box fits)
constexpr int FC_GROUP = 8;                     // pairs per group: one per 8-lane row
constexpr int FC_LISTCAP = FC_GROUP * FC_TCAP;  // a group's survivors always fit: no overflow handling
constexpr int FC_SHIFT = 7;                     // list entry = pair-in-group << 7 | table index
constexpr int FC_BIGSHIFT = 13;                 // ... of an item of several chunks: pair-in-group << 13 | index in its box
constexpr int FC_BIGT = 1 << FC_BIGSHIFT;       // (boxes of up to 8192 translations)
#ifndef CFH_NORD
#define CFH_NORD 5
#endif
constexpr int NORD = CFH_NORD;                  // moments per axis
constexpr int CORE_WPB = 1;                     // wavefronts per workgroup of the main kernels: each takes an item of its
                                                // own (no barriers).  Workgroups of 4 or 8 items of one head that make the
                                                // products with the head's weights themselves (projection, G) were slower:
                                                // +25 us per kernel for the phases behind barriers, against 21 + 20 us for
                                                // the two separate launches
constexpr int FC_LOGCAP = 64;                   // logits of a row kept in LDS until the row is complete
constexpr int HW_DIST = NBINS;
constexpr int HW_ANG = NBINS * (1 + 3 * NORD);  // 1024 words per (atom, head) with the 64-bin angle encoding
constexpr int SMALL_A = 16;                     // the 16-bin angle basis (the reference's lightweight setting): sigma is
                                                // one bin or more, far too wide a step for the moment series, and the
                                                // basis is small: every image adds its 16 basis values per axis directly
                                                // (the whole basis, as the reference evaluates it for 16 bins)
constexpr int HW_ANG16 = 2 * NBINS;             // 64 distance bins + 3 axes x 16 bins, padded to whole 64-word blocks
// In LDS the 3 x 16 angle bins of an item exist A16_COPIES times, one copy per value of lane & 15: every image adds
// to ALL 16 bins of an axis in the same order, so with one copy the 64 lanes of an atomic instruction would meet on
// one word (128 clocks instead of 6).  A copy has an odd number of words so that the copies start in different banks.
constexpr int A16_COPIES = 16;
constexpr int A16_STRIDE = 3 * SMALL_A + 1;
// words of an item's histogram in LDS
__host__ __device__ constexpr int core_hist_lds_words(int ang) {
    return ang == SMALL_A ? HW_DIST + A16_COPIES * A16_STRIDE : (ang == NBINS ? HW_ANG : HW_DIST);
}
// words of an item's histogram for `ang` angle bins (0: distance encoding alone)
__host__ __device__ constexpr int core_hist_words(int ang) { return ang == NBINS ? HW_ANG : (ang == SMALL_A ? HW_ANG16 : HW_DIST); }
constexpr int REC_J0 = 30;                      // item record: first neighbour atom (pairs of an atom are j0, j0+1, ...)
constexpr int REC_CRYSTAL = 31;                 // item record: crystal of the atom
static_assert(FC_TCAP == (1 << FC_SHIFT) && (FC_GROUP << FC_SHIFT) <= 65536, "list entry is 16 bits");

typedef float v4f_c __attribute__((ext_vector_type(4)));

// Optional phase timing (compile with -DCFH_PHASE_TIMING; diagnostics builds only): cycles per phase of the forward
// kernel, summed over the wavefronts, in the statistics slots 16..23.
#ifdef CFH_PHASE_TIMING
#define CFH_PH_DECL unsigned long long ph_acc[8] = {0, 0, 0, 0, 0, 0, 0, 0}; unsigned long long ph_last = __builtin_amdgcn_s_memtime(); int ph_cur = 0;
#define CFH_PH(n) do { const unsigned long long ph_t = __builtin_amdgcn_s_memtime(); ph_acc[ph_cur] += ph_t - ph_last; ph_last = ph_t; ph_cur = (n); } while (0)
#define CFH_PH_FLUSH(stats) do { CFH_PH(0); if ((stats) && (threadIdx.x & 63) == 0) for (int u = 0; u < 8; u++) atomicAdd((stats) + 16 + u, ph_acc[u]); } while (0)
#else
#define CFH_PH_DECL
#define CFH_PH(n) do { } while (0)
#define CFH_PH_FLUSH(stats) do { } while (0)
#endif

struct CoreArgs {
    KernelArgs K;                 // geometry, work queues, item records, basis constants
    const float* qs;              // (N,H,16) query, already divided by sqrt(16)
    const float* k;               // (N,H,16)
    const float* v;               // (N,H,16)
    const float4* sorted_tab;     // (B, FC_TCAP) shifts of the usual box sorted by length, w = length; or null
    const float2* pair_near;      // (E) per pair over that box: smallest d^2 of all images, of the images with
                                  // d^2 > 1e-5 (what the frame search may point at; low 7 bits: that image's
                                  // position in the sorted table); or null
    int32_t table_R;              // half-width that table was made for
    int32_t slow_wgs;             // leading wavefronts of the main kernels that take the listed slow records first, by
                                  // rank over all lists: wavefront w the rank w; the listed records of higher rank are
                                  // taken in place, like the others (0: no lists)
    int32_t slow_lists;           // lists (K.slow_count, K.slow_list)
    int32_t slow_stride;          // slots per list
    uint32_t slow_flag;           // the flag in the box word of the records listed for this launch
    float skip_log2;              // images lighter than 2^-skip of the heaviest of their pair are not visited (<= 0: all are)
    // forward results
    float* out;                   // (N,H,16) sum_j P_ij v_j (core_project_kernel adds W . hist)
    float* prob;                  // (E,H) P_ij
    float* z;                     // (E,H)
    float* hist;                  // (H,N,hw)
    // backward operands and results
    const float* go;              // (N,H,16) upstream gradient of out
    const float* outv;            // (N,H,16) the forward's final out
    const float* G;               // (H,N,hw) Wcat^T go per item
    float* gq;                    // (N,H,16)
    float* glogit;                // (E,H) gradient of the logits (the column kernel turns it into gk)
};

// Loads at a 32-bit BYTE offset from a base that is the same in all lanes: the address is (scalar base + vector offset),
// one instruction's operands, where an element index of 64 bits costs two or three vector instructions per address
// (the entry points refuse sizes whose offsets would not fit).
template <typename T>
__device__ __forceinline__ T load_at(const void* base, uint32_t byte_off) {
    return *reinterpret_cast<const T*>(reinterpret_cast<const char*>(base) + byte_off);
}

// ---- reductions over an 8-lane row (half of a DPP row) -------------------------------------------------------
__device__ __forceinline__ float half_sum(float x) {
    x += dpp_move<0xB1>(x); x += dpp_move<0x4E>(x); x += dpp_move<0x141>(x); return x;
}
__device__ __forceinline__ float half_min(float x) {
    x = fminf(x, dpp_move<0xB1>(x)); x = fminf(x, dpp_move<0x4E>(x)); x = fminf(x, dpp_move<0x141>(x)); return x;
}
__device__ __forceinline__ float wave_maxf(float v) { return -wave_min(-v); }
// sum over the 8 rows for every position in the row: lanes s, s+8, ..., s+56
__device__ __forceinline__ float rows8_sum(float x) {
    x += dpp_move<0x128>(x);          // row_ror 8: the other half of the 16-lane row
    return rows_sum(x);
}
// float -> fixed point, round to nearest (floor(x + 0.5)) in ONE instruction (rintf + conversion are two)
__device__ __forceinline__ int rint_i(float x) {
    int r;
    asm("v_cvt_rpi_i32_f32 %0, %1" : "=v"(r) : "v"(x));
    return r;
}

// ---- sorted shifts of the usual box, one table per crystal ---------------------------------------------------
// block = crystal, 128 threads; entry = (shift, |shift|), ascending length (ties: loop order); entries beyond the
// box: length +inf.  The low 7 bits of the length hold the translation's index in the reference's loop order (the
// frame search breaks ties by it): the length is rounded down by at most 2^-16 of itself, which the margins of every
// reach test cover.
__global__ __launch_bounds__(FC_TCAP) void sorted_shifts_kernel(const float* __restrict__ tvecs, int R0, float4* __restrict__ out) {
    __shared__ float key[FC_TCAP];
    const int b = blockIdx.x, t = threadIdx.x;
    const int s = 2 * R0 + 1, T0 = s * s * s;
    float4 v = make_float4(0.f, 0.f, 0.f, __builtin_inff());
    if (t < T0) {
        const float* L = tvecs + (size_t)b * 9;
        const float n3 = (float)(t % s - R0), n2 = (float)((t / s) % s - R0), n1 = (float)(t / (s * s) - R0);
        v.x = fmaf(L[6], n3, fmaf(L[3], n2, L[0] * n1));
        v.y = fmaf(L[7], n3, fmaf(L[4], n2, L[1] * n1));
        v.z = fmaf(L[8], n3, fmaf(L[5], n2, L[2] * n1));
        v.w = sqrtf(fmaf(v.x, v.x, fmaf(v.y, v.y, v.z * v.z)));
    }
    key[t] = v.w;
    __syncthreads();
    int rank = 0;
    for (int u = 0; u < FC_TCAP; u++) {
        const float ku = key[u];
        rank += (ku < v.w || (ku == v.w && u < t)) ? 1 : 0;
    }
    if (t < T0) v.w = __uint_as_float((__float_as_uint(v.w) & ~(uint32_t)(FC_TCAP - 1)) | (uint32_t)t);
    out[(size_t)b * FC_TCAP + rank] = v;
}

// Per pair, over the usual box of its crystal: the smallest squared distance of all images and of the images with
// d^2 > 1e-5, the latter with the position of that image in the sorted table in its low 7 bits.  Both depend on the geometry alone, not on the head or the layer, so they are made once per batch:
// the lattice sums of an item with the usual box then need no sweep for the nearest image, and the frame search
// knows how far into the sorted table a pair's best first-axis candidate can sit.  Eight lanes per pair, eight
// entries of the sorted table at a time; the sorted order ends the loop once |s| - |r| exceeds the larger of the
// two minima (an entry behind that point cannot lower either minimum, so taking the rest of its group of eight
// along changes nothing).  Same arithmetic for d^2 as the sweeps.  A thread per pair walking the table alone took
// 16 us for its chain of dependent steps; this takes 7.
__global__ __launch_bounds__(256) void pair_nearest_kernel(const float* __restrict__ rpos, const int64_t* __restrict__ edges,
                                                           const int64_t* __restrict__ batch,
                                                           const float4* __restrict__ sorted_tab, int T0, int E,
                                                           float2* __restrict__ out) {
    const int g = blockIdx.x * blockDim.x + threadIdx.x;
    const int e = min(g >> 3, E - 1), sub = g & 7;       // (the lanes of a group past the end redo the last pair)
    const int b = (int)batch[edges[e]];
    const float4* tab = sorted_tab + (size_t)b * FC_TCAP;
    const float rx = rpos[(size_t)e * 3 + 0], ry = rpos[(size_t)e * 3 + 1], rz = rpos[(size_t)e * 3 + 2];
    const float r = sqrtf(fmaf(rx, rx, fmaf(ry, ry, rz * rz)));
    // (dval carries the table position of its image in its low 7 bits -- it is rounded down by at most 2^-16 of itself,
    // which the margins of every test that uses it cover -- so that the minimum over the lanes brings the position along)
    float dall = 3.0e38f, dval = 3.0e38f;
    for (int t0 = 0; t0 < T0; t0 += 8) {
        // the first entry of the group decides for all eight lanes whether the walk goes on
        if (dval < 1.0e38f && tab[t0].w > fmaf(1.0001f, r + sqrtf(dval), 1e-3f)) break;
        if (t0 + sub < T0) {
            const float4 v = tab[t0 + sub];
            const float dx = rx + v.x, dy = ry + v.y, dz = rz + v.z;
            const float d2 = fmaf(dx, dx, fmaf(dy, dy, dz * dz));
            dall = fminf(dall, d2);
            if (d2 > 1e-5f)
                dval = fminf(dval, __uint_as_float((__float_as_uint(d2) & ~(uint32_t)(FC_TCAP - 1)) | (uint32_t)(t0 + sub)));
        }
        dall = half_min(dall);
        dval = half_min(dval);
    }
    if (sub == 0 && (g >> 3) < E) out[e] = make_float2(dall, dval);
}

// ---- projection weights with the moment matrices folded in ---------------------------------------------------
// D_o(d) = exp(-(d/ws)^2/2) He_o(d/ws) / (o! (2 ws)^o)
__device__ __forceinline__ float moment_matrix(int o, float d, float ws) {
    const float y = d / ws;
    float h0 = 1.0f, h1 = y;           // probabilists' Hermite polynomials
    float he = o == 0 ? h0 : h1;
    for (int n = 1; n < o; n++) { const float h2 = y * h1 - (float)n * h0; h0 = h1; h1 = h2; he = h2; }
    float coef = 1.0f;
    for (int n = 1; n <= o; n++) coef /= (float)n * 2.0f * ws;
    return __expf(-0.5f * y * y) * he * coef;
}
// table of D_o(d) for d = -63 .. 63 in LDS, made by the 256 threads of a block: dtab[o * 128 + d + 63]
__device__ __forceinline__ void build_moment_table(float* dtab, float ws) {
    for (int u = threadIdx.x; u < NORD * 128; u += 256) {
        const int o = u >> 7, d = (u & 127) - 63;
        dtab[u] = (u & 127) < 127 ? moment_matrix(o, (float)d, ws) : 0.0f;
    }
    __syncthreads();
}
// wcat (H,16,hw): [0,64) dist_coef W_dist;  64 + (ax NORD + o) 64 + m': angle_coef sum_m W_ax[c,m] D_o(m - m').
// grid: H*16 blocks (h, c), 256 threads over the words.
struct WcatArgs {
    const float* Wd; const float* W1; const float* W2; const float* W3;      // (H,16,64) and (H,16,A) x 3
    int hw;
    float dist_coef, angle_coef, ws;
    float* wcat;
};
__device__ __forceinline__ void core_wcat_block(const WcatArgs& A, int hc) {
    const float* __restrict__ Wd = A.Wd; const float* __restrict__ W1 = A.W1;
    const float* __restrict__ W2 = A.W2; const float* __restrict__ W3 = A.W3;
    const int hw = A.hw;
    const float dist_coef = A.dist_coef, angle_coef = A.angle_coef, ws = A.ws;
    float* __restrict__ wcat = A.wcat;
    __shared__ float row[3][NBINS];
    __shared__ float dtab[NORD * 128];
    if (hw == HW_ANG16) {
        // 16-bin basis: the weights themselves behind the distance block, zeros in the padding
        for (int w = threadIdx.x; w < hw; w += 256) {
            float val = 0.0f;
            if (w < HW_DIST) val = dist_coef * Wd[(size_t)hc * NBINS + w];
            else if (w < HW_DIST + 3 * SMALL_A) {
                const int u = w - HW_DIST, ax = u / SMALL_A, m = u % SMALL_A;
                const float* W = ax == 0 ? W1 : (ax == 1 ? W2 : W3);
                val = angle_coef * W[(size_t)hc * SMALL_A + m];
            }
            wcat[(size_t)hc * hw + w] = val;
        }
        return;
    }
    if (hw > HW_DIST) {
        for (int u = threadIdx.x; u < 3 * NBINS; u += 256) {
            const float* W = u < NBINS ? W1 : (u < 2 * NBINS ? W2 : W3);
            row[u / NBINS][u % NBINS] = W[(size_t)hc * NBINS + (u % NBINS)];
        }
        build_moment_table(dtab, ws);
    }
    for (int w = threadIdx.x; w < hw; w += 256) {
        float val;
        if (w < HW_DIST) val = dist_coef * Wd[(size_t)hc * NBINS + w];
        else {
            const int u = w - HW_DIST, ax = u / (NORD * NBINS), o = (u / NBINS) % NORD, mp = u % NBINS;
            const float* dt = dtab + o * 128 + 63 - mp;
            float acc = 0.0f;
#pragma unroll 8
            for (int m = 0; m < NBINS; m++) acc = fmaf(row[ax][m], dt[m], acc);
            val = angle_coef * acc;
        }
        wcat[(size_t)hc * hw + w] = val;
    }
}
__global__ __launch_bounds__(256) void core_wcat_kernel(const WcatArgs A) { core_wcat_block(A, (int)blockIdx.x); }
// The item records of a launch and the concatenated weights in ONE launch (neither depends on the other; both are a
// few microseconds of work behind a launch): the first prep_blocks workgroups are those of prepare_items_kernel, the
// following H * 16 those of core_wcat_kernel.
__global__ __launch_bounds__(256) void core_prepare_wcat_kernel(const KernelArgs P, int with_query, int prep_blocks,
                                                                const WcatArgs A) {
    if ((int)blockIdx.x < prep_blocks) prepare_items_block(P, with_query, (int)blockIdx.x);
    else core_wcat_block(A, (int)blockIdx.x - prep_blocks);
}
// The way back: gW_dist = dist_coef gwcat[.., 0:64];  gW_ax[c,m] = angle_coef sum_{o,m'} gwcat[.., ax,o,m'] D_o(m - m').
// Block hc = (head, channel), 256 threads = (enc 0..3, bin m).  ACC: added to what the destinations hold.
template <bool ACC>
__device__ __forceinline__ void core_gw_finish_block(const float* __restrict__ gwcat, int nslices, size_t slice_stride,
                                                     int hw, float dist_coef, float angle_coef, float ws,
                                                     float* __restrict__ gWd, float* __restrict__ gW1,
                                                     float* __restrict__ gW2, float* __restrict__ gW3, int hc) {
    __shared__ float dtab[NORD * 128];
    __shared__ float grow[3 * NORD * NBINS];
    const int enc = threadIdx.x >> 6, m = threadIdx.x & 63;
    const float* g = gwcat + (size_t)hc * hw;
    if (hw == HW_ANG16) {
        // 16-bin basis: thread (enc, m) sums the slices of its word; the axes' rows have 16 bins
        if (enc > 0 && m >= SMALL_A) return;
        float* dst = enc == 0 ? gWd : (enc == 1 ? gW1 : (enc == 2 ? gW2 : gW3));
        if (!dst) return;
        const int word = enc == 0 ? m : HW_DIST + (enc - 1) * SMALL_A + m;
        float sum = 0.0f;
        for (int sl = 0; sl < nslices; sl++) sum += g[sl * slice_stride + word];      // fixed order
        float* d = dst + (size_t)hc * (enc == 0 ? NBINS : SMALL_A) + m;
        *d = (ACC ? *d : 0.0f) + (enc == 0 ? dist_coef : angle_coef) * sum;
        return;
    }
    if (hw > HW_DIST) {
        for (int u = threadIdx.x; u < 3 * NORD * NBINS; u += 256) {
            float sum = 0.0f;
            for (int sl = 0; sl < nslices; sl++) sum += g[sl * slice_stride + HW_DIST + u];      // fixed order
            grow[u] = sum;
        }
        build_moment_table(dtab, ws);
    }
    if (enc == 0) {
        if (gWd) {
            float sum = 0.0f;
            for (int sl = 0; sl < nslices; sl++) sum += g[sl * slice_stride + m];
            float* d = gWd + (size_t)hc * NBINS + m;
            *d = (ACC ? *d : 0.0f) + dist_coef * sum;
        }
        return;
    }
    if (hw <= HW_DIST) return;
    float* dst = enc == 1 ? gW1 : (enc == 2 ? gW2 : gW3);
    if (!dst) return;
    float acc = 0.0f;
    for (int o = 0; o < NORD; o++) {
        const float* gr = grow + ((enc - 1) * NORD + o) * NBINS;
        const float* dt = dtab + o * 128 + 63 + m;
#pragma unroll 8
        for (int mp = 0; mp < NBINS; mp++) acc = fmaf(gr[mp], dt[-mp], acc);
    }
    float* d = dst + (size_t)hc * NBINS + m;
    *d = (ACC ? *d : 0.0f) + angle_coef * acc;
}
// grid: H*16 blocks.
__global__ __launch_bounds__(256) void core_gw_finish_kernel(const float* __restrict__ gwcat, int nslices, int H, int hw,
                                                             float dist_coef, float angle_coef, float ws,
                                                             float* __restrict__ gWd, float* __restrict__ gW1,
                                                             float* __restrict__ gW2, float* __restrict__ gW3) {
    core_gw_finish_block<false>(gwcat, nslices, (size_t)H * DH * hw, hw, dist_coef, angle_coef, ws, gWd, gW1, gW2, gW3,
                                (int)blockIdx.x);
}

// Weight gradients of several calls of the core (the layers of a backward pass) in one launch each way.
constexpr int CORE_WG_MAX_JOBS = 8;
constexpr int CORE_GW_SLICES = 8;      // at most this many slices of the atoms per job (copies of the scratch)
struct CoreWgradJob {
    const float* go;       // (N,H,16)
    const float* hist;     // (H,N,hw)
    float* gwcat;          // (nslices,H,16,hw) scratch
    float* gW[4];          // destinations (H,16,64), added to; null: not wanted
    int N, per_slice, slice0, nslices;      // atoms, atoms per slice, first slice (blockIdx.z) of this job, its slices
};
struct CoreWgradJobs {
    CoreWgradJob job[CORE_WG_MAX_JOBS];
    int njobs, H, hw;
    float dist_coef, angle_coef, ws;
};
// ---- distance window with round-to-nearest fixed-point adds ---------------------------------------------------
template <int W>
__device__ __forceinline__ void window_scatter_rn(int32_t* base, const WindowSeed& s, float cc, int wrt = 0) {
    const int Wd = W > 0 ? W : wrt, C = Wd / 2;      // (W == 0: the width is known at run time only)
    atomicAdd(base + C, rint_i(s.gc));
    float g = s.gc, r = s.rr;
#pragma unroll
    for (int m = C + 1; m < Wd; m++) { g *= r; r *= cc; atomicAdd(base + m, rint_i(g)); }
    g = s.gc; r = s.rl;
#pragma unroll
    for (int m = C - 1; m >= 0; m--) { g *= r; r *= cc; atomicAdd(base + m, rint_i(g)); }
}

// ---- shared pieces of the two main kernels ---------------------------------------------------------------------
struct CoreItem {
    Item item;
    int j0, crystal;
    bool sorted;
    int nchunks;
};
__device__ __forceinline__ CoreItem core_unpack(const CoreArgs& C, uint32_t rec, bool want_sorted) {
    CoreItem ci;
    ci.item = unpack_item(rec);
    ci.j0 = __builtin_amdgcn_readlane((int)rec, REC_J0);
    ci.crystal = __builtin_amdgcn_readlane((int)rec, REC_CRYSTAL);
    const Box& bx = ci.item.bx;
    ci.sorted = want_sorted && C.sorted_tab != nullptr && bx.R1 == C.table_R && bx.R2 == C.table_R &&
                bx.R3 == C.table_R && ci.item.a < 0.0f && C.skip_log2 > 0.0f;
    ci.nchunks = ci.sorted ? 1 : (bx.T + FC_TCAP - 1) / FC_TCAP;
    return ci;
}
// table of the item's first (or only) chunk
// build_shift_table with the rest of the last group of FC_GROUP entries filled with length +inf: a sweep then needs
// one comparison per entry, length <= limit, for "inside the table", "the row has a pair" and "within reach" together
// (the sorted tables end in such entries as well; built tables have length 0 in every real entry).
__device__ __forceinline__ void build_shift_table_padded(float4* tab, int t0, int cnt, const Box& bx, const Lattice& L,
                                                         int lane) {
    build_shift_table(tab, t0, cnt, bx, L, lane);
    const int u = cnt + lane;
    if (lane < 8 && u < ((cnt + 7) & ~7)) tab[u] = make_float4(0.f, 0.f, 0.f, __builtin_inff());
}
constexpr float FC_REACH_ALL = 3.0e38f;       // a reach that every real entry is within, and no padding entry

__device__ __forceinline__ void core_load_table(const CoreArgs& C, const CoreItem& ci, float4* tab, int lane) {
    if (ci.sorted) {
        for (int u = lane; u < FC_TCAP; u += WAVE) tab[u] = C.sorted_tab[(size_t)ci.crystal * FC_TCAP + u];
    } else if (ci.nchunks == 1) {
        build_shift_table_padded(tab, 0, ci.item.bx.T, ci.item.bx, ci.item.L, lane);
    }
}

// Operands of an item that do not depend on the item before it, fetched a whole item ahead: the two table entries
// of this lane (sorted table of the item's crystal), the lane's two query channels, and the operands of the pair
// of the first group that this lane's row serves.
struct CorePrefetch {
    float4 t0, t1;
    float2 q2;
    float rx, ry, rz;
    float2 k2, v2;
    float near;       // smallest d^2 over the images of that pair (when the batch's table of them is given)
};
__device__ __forceinline__ CorePrefetch core_prefetch(const CoreArgs& C, uint32_t rec, int it, int h, int lane) {
    CorePrefetch pf;
    pf.t0 = pf.t1 = make_float4(0.f, 0.f, 0.f, 0.f);
    pf.q2 = pf.k2 = pf.v2 = make_float2(0.f, 0.f);
    pf.rx = pf.ry = pf.rz = 0.f;
    pf.near = 3.0e38f;
    if (it < 0) return pf;
    const KernelArgs& P = C.K;
    const int H = P.H;
    const int i = __builtin_amdgcn_readlane((int)rec, REC_ATOM);
    const int e0 = __builtin_amdgcn_readlane((int)rec, REC_E0);
    const int npairs = __builtin_amdgcn_readlane((int)rec, REC_NPAIRS);
    const int j0 = __builtin_amdgcn_readlane((int)rec, REC_J0);
    const int crystal = __builtin_amdgcn_readlane((int)rec, REC_CRYSTAL);
    const int pr = lane >> 3, sub = lane & 7;
    if (C.sorted_tab) {
        const float4* src = C.sorted_tab + (size_t)crystal * FC_TCAP;
        pf.t0 = src[lane];
        pf.t1 = src[lane + WAVE];
    }
    pf.q2 = load_at<float2>(C.qs, (((uint32_t)i * (uint32_t)H + (uint32_t)h) * DH + 2u * sub) * 4u);
    if (npairs > 0) {
        // (no branch per row: a row past the end re-reads the row's last pair; nothing of it is used)
        const uint32_t el = (uint32_t)min(pr, npairs - 1);
        const uint32_t e = min((uint32_t)e0 + el, (uint32_t)(P.E - 1));
        const uint32_t jh = ((((uint32_t)j0 + el) * (uint32_t)H + (uint32_t)h) * DH + 2u * sub) * 4u;
        const float3 r3 = load_at<float3>(P.rpos, e * 12u);
        pf.rx = r3.x; pf.ry = r3.y; pf.rz = r3.z;
        pf.k2 = load_at<float2>(C.k, jh);
        pf.v2 = load_at<float2>(C.v, jh);
        if (C.pair_near) pf.near = load_at<float>(C.pair_near, e * 8u);
    }
    return pf;
}
// the item's table from what was prefetched (sorted) or built in place (one chunk)
__device__ __forceinline__ void core_store_table(const CoreItem& ci, const CorePrefetch& pf, float4* tab, int lane) {
    if (ci.sorted) {
        tab[lane] = pf.t0;
        tab[lane + WAVE] = pf.t1;
    } else if (ci.nchunks == 1) {
        build_shift_table_padded(tab, 0, ci.item.bx.T, ci.item.bx, ci.item.L, lane);
    }
}

// The record of rank r over the slow lists (list after list, a list's records in order), or -1 past the last; r is
// the same in all lanes.  Two levels, so that the wavefront waits for memory twice whatever the number of lists: every
// lane adds the counts of its own run of consecutive lists (loads that do not depend on each other), a prefix sum over
// the lanes names the run that holds rank r, and a second prefix sum over the counts of that run names the list.
__device__ __forceinline__ int core_slow_record(const CoreArgs& C, int r, int lane) {
    const int n = C.slow_lists;
    const int run = (n + WAVE - 1) / WAVE;
    int mine = 0;
    for (int k = 0; k < run; k++) mine += lane * run + k < n ? C.K.slow_count[lane * run + k] : 0;
    const int incl = wave_scan_incl(mine);
    if (r >= __builtin_amdgcn_readlane(incl, WAVE - 1)) return -1;
    const int seg = __builtin_amdgcn_readfirstlane(__ffsll((unsigned long long)ballot(incl > r)) - 1);
    int base = __builtin_amdgcn_readlane(incl - mine, seg);
    for (int k0 = 0; k0 < run; k0 += WAVE) {
        const int li = seg * run + k0 + lane;
        const int c = (k0 + lane < run && li < n) ? C.K.slow_count[li] : 0;
        const int inc2 = wave_scan_incl(c);
        const int tot = __builtin_amdgcn_readlane(inc2, WAVE - 1);
        if (r < base + tot) {
            const int l = __builtin_amdgcn_readfirstlane(__ffsll((unsigned long long)ballot(base + inc2 > r)) - 1);
            const int excl = __builtin_amdgcn_readlane(inc2 - c, l);
            return C.K.slow_list[(size_t)(seg * run + k0 + l) * C.slow_stride + (r - base - excl)];
        }
        base += tot;
    }
    return -1;
}
// Which record a wavefront of a main kernel starts with: the first slow_wgs wavefronts a listed one (-1: none left),
// the others the records in work order.
__device__ __forceinline__ int core_wave_record(const CoreArgs& C, int w, int lane) {
    // (the same in all lanes: said so, the index arithmetic that follows stays on the scalar unit)
    return __builtin_amdgcn_readfirstlane(w < C.slow_wgs ? core_slow_record(C, w, lane) : w - C.slow_wgs);
}
// The rank over the slow lists of the listed record `wid`: the counts of the lists before its own, and its place in its
// own list (records in ascending order: the entries below it).
__device__ __forceinline__ int core_slow_rank(const CoreArgs& C, int wid, int lane) {
    const int li = wid / C.slow_stride;
    int part = 0;
    for (int c0 = lane; c0 < li; c0 += WAVE) part += C.K.slow_count[c0];
    const int n = C.K.slow_count[li];
    const int32_t* lst = C.K.slow_list + (size_t)li * C.slow_stride;
    for (int k = lane; k < n; k += WAVE) part += lst[k] < wid ? 1 : 0;
    return __builtin_amdgcn_readlane(wave_scan_incl(part), WAVE - 1);
}
// A listed record is left to the leading wavefront of its rank; ranks past the leading wavefronts stay in place.
// `wave_id`: this wavefront's number in the launch.
__device__ __forceinline__ bool core_record_taken_elsewhere(const CoreArgs& C, uint32_t rec, int wid, int lane) {
    if (C.slow_wgs == 0 || (int)(blockIdx.x * CORE_WPB + (threadIdx.x >> 6)) < C.slow_wgs) return false;
    if (((uint32_t)__builtin_amdgcn_readlane((int)rec, REC_BOX) & C.slow_flag) == 0u) return false;
    return core_slow_rank(C, wid, lane) < C.slow_wgs;
}

// =================================================================================================================
// forward
// =================================================================================================================
template <int HWK>
struct CoreFwdShared {
    float4 tab[FC_TCAP];
    uint16_t list[FC_LISTCAP];
    int32_t hist[HWK];
    float4 pairA[FC_GROUP];      // rx, ry, rz, d2min
    float pairC[FC_GROUP];       // exp(logit - running max) / S in fixed-point units
    float logit_s[FC_LOGCAP];    // logits of the row (rows of more pairs park them in the probability array)
};
template <int WL, int ANG, bool COS_ABS>
// ANG: angle bins, 0 (distance encoding alone), 64 (moment series) or 16 (basis values added directly)
// (distance encoding alone: 4.8 KB of LDS per item allow eight wavefronts per SIMD; seven, with 72 registers and
// nothing spilled, ran faster than eight with 64 and nine spilled)
__global__ __launch_bounds__(WAVE * CORE_WPB) __attribute__((amdgpu_waves_per_eu(ANG > 0 ? 1 : 7)))
void fused_core_fwd_kernel(const CoreArgs C) {
    constexpr bool HAS_ANG = ANG > 0;
    constexpr int HWK = core_hist_words(ANG);          // words per item in memory
    constexpr int HWL = core_hist_lds_words(ANG);      // ... and in LDS
    constexpr bool VEC = HWL == HWK && HWK >= 4 * WAVE;      // clear, rescale and store four words per lane at a time
    __shared__ CoreFwdShared<HWL> shared[CORE_WPB];
    CoreFwdShared<HWL>& sh = shared[threadIdx.x >> 6];
    float4* const tab = sh.tab;
    uint16_t* const list = sh.list;
    int32_t* const hist = sh.hist;
    float4* const pairA = sh.pairA;
    float* const pairC = sh.pairC;
    float* const logit_s = sh.logit_s;

    const KernelArgs& P = C.K;
    const int lane = threadIdx.x & (WAVE - 1);
    const int H = P.H;
    const int wid = core_wave_record(C, (int)blockIdx.x * CORE_WPB + (int)(threadIdx.x >> 6), lane);      // this wavefront's (item, head)
    if (wid < 0) return;
    const int it_cur = div_heads(P, wid);      // items in descending order of their pair count: the long ones start first
    const int h = wid - it_cur * H;
    const int pr = lane >> 3;          // pair of the group served by this 8-lane row
    const int sub = lane & 7;          // position in the row
    const BasisConsts bc = P.bc;
    const int WLr = WL > 0 ? WL : bc.len_window;      // bins of the distance window (WL == 0: known at run time only)
    const float prune = (P.prune_log2 > 0.0f) ? -P.prune_log2 : -3.0e38f;
    const float INF = __builtin_inff();

    if (it_cur >= P.N) return;
    if (VEC) {
#pragma unroll
        for (int u = 0; u < HWK / (4 * WAVE); u++) reinterpret_cast<int4*>(hist)[lane + WAVE * u] = make_int4(0, 0, 0, 0);
    } else {
        for (int u = lane; u < HWL; u += WAVE) hist[u] = 0;
    }
    wave_sync();

    CFH_PH_DECL
    {
        const uint32_t rec_cur = load_record_lane(P, it_cur, h, lane);
        if (core_record_taken_elsewhere(C, rec_cur, wid, lane)) return;
        const CorePrefetch pf = core_prefetch(C, rec_cur, it_cur, h, lane);
        CFH_PH(0);
        const CoreItem ci = core_unpack(C, rec_cur, true);
        const int i = ci.item.i;
        const float a = ci.item.a;
        const float a2 = a * LOG2E;
        const Lattice L = ci.item.L;
        const Box bx = ci.item.bx;
        const bool sorted = ci.sorted;
        const int nchunks = ci.nchunks;
        float f[3][3];
        if (HAS_ANG) {
#pragma unroll
            for (int ax = 0; ax < 3; ax++)
#pragma unroll
                for (int d = 0; d < 3; d++) f[ax][d] = rec_f(rec_cur, REC_FRAMES + ax * 3 + d);
        }
        const int e0 = ci.item.e0, npairs = ci.item.npairs;
        wave_sync();                          // the previous item's readers of the table are done
        core_store_table(ci, pf, tab, lane);
        wave_sync();
        const size_t ih = (size_t)i * H + h;
        const float2 q2 = pf.q2;
        // 2^30 / npairs: sums of weights <= 1 each fit (hardware reciprocal: any scale near it will do, the histogram
        // is divided by the same number when it is written)
        const float fixs = 1073741824.0f * hw_rcp((float)max(npairs, 1));
        const float cutS = (C.skip_log2 > 0.0f && a2 < 0.0f) ? C.skip_log2 * hw_rcp(-a2) : INF;      // (a bound with margins)
        float m_run = -INF;                   // running maximum of the logits (wave-uniform)
        float Dl = 0.0f;                      // this lane's share of the softmax denominator
        float2 accv = make_float2(0.f, 0.f);  // sum_j exp(logit_j - m_run) v_j, channels 2 sub, 2 sub + 1
        unsigned long long n_eval = 0, n_seen = 0;      // wave-uniform counts

        // operands of the pair served by this row, fetched one group ahead (the first group: with the item)
        float nrx = pf.rx, nry = pf.ry, nrz = pf.rz, nnear = pf.near;
        float2 nk2 = pf.k2, nv2 = pf.v2;
        // The nearest image of every pair over the usual box comes with the batch.  An item whose box CONTAINS the usual
        // one takes it as the reference of its weights as well (any reference gives the same normalised weights and
        // the same z; only the pruning threshold moves with it, should an image outside the usual box be nearer)
        const bool contains_usual = C.sorted_tab != nullptr && bx.R1 >= C.table_R && bx.R2 >= C.table_R && bx.R3 >= C.table_R;
        const bool near_known = (sorted || contains_usual) && C.pair_near != nullptr;
        // several chunks: the survivors of all chunks go into one list with their index in the whole box, and the
        // heavy pass makes their shifts from that index instead of reading a table: one sweep, each chunk built once
        const bool one_list = nchunks > 1 && bx.T <= FC_BIGT;
        auto fetch = [&](int g0) {
            // (no branch per row: a row past the end re-reads the row's last pair; nothing of it is used)
            const uint32_t el = (uint32_t)min(g0 + pr, npairs - 1);
            const uint32_t e = min((uint32_t)e0 + el, (uint32_t)(P.E - 1));
            const uint32_t jh = ((((uint32_t)ci.j0 + el) * (uint32_t)H + (uint32_t)h) * DH + 2u * sub) * 4u;
            const float3 r3 = load_at<float3>(P.rpos, e * 12u);
            nrx = r3.x; nry = r3.y; nrz = r3.z;
            nk2 = load_at<float2>(C.k, jh);
            nv2 = load_at<float2>(C.v, jh);
            if (near_known) nnear = load_at<float>(C.pair_near, e * 8u);
        };

        // one sweep of this row's pair over the table(s): fn(inside, index in the chunk, first index of the chunk, d^2, rows inside)
        auto sweep = [&](bool active, float rx, float ry, float rz, float reach, auto&& fn) {
            const float lim = active ? fminf(reach, FC_REACH_ALL) : -1.0f;      // (lengths are >= 0; padding: +inf)
            for (int ch = 0; ch < nchunks; ch++) {
                const int t0c = ch * FC_TCAP;
                const int cnt = sorted ? bx.T : min(FC_TCAP, bx.T - t0c);
                if (nchunks > 1) {
                    wave_sync();
                    build_shift_table_padded(tab, t0c, cnt, bx, L, lane);
                    wave_sync();
                }
                float4 v = tab[sub];
                for (int t0 = 0; t0 < cnt; t0 += FC_GROUP) {
                    const int t = t0 + sub;
                    const float4 vn = tab[min(t + FC_GROUP, FC_TCAP - 1)];      // the next step's entry, in flight meanwhile
                    const bool in = v.w <= lim;
                    const uint64_t inm = ballot(in);
                    if (sorted && inm == 0) break;               // every row is past its reach (lengths ascend)
                    const float dx = rx + v.x, dy = ry + v.y, dz = rz + v.z;
                    fn(in, t, t0c, fmaf(dx, dx, fmaf(dy, dy, dz * dz)), __popcll(inm));
                    v = vn;
                }
            }
        };

        // scatter of the current list (entries point into the resident table)
        auto heavy_impl = [&](int nlist, auto big) {
            constexpr bool BIG = decltype(big)::value;      // entries (pair << FC_BIGSHIFT | index in the box), no table
            // (hardware reciprocals, within an ulp: the quotients below stay exact all the same)
            const float inv_s3 = BIG ? hw_rcp((float)bx.s3) : 0.0f, inv_s2 = BIG ? hw_rcp((float)bx.s2) : 0.0f;
            for (int base = 0; base < nlist; base += WAVE) {
                const int idx = base + lane;
                if (idx < nlist) {
                    const uint32_t ent = list[idx];
                    const int pp = BIG ? (int)(ent >> FC_BIGSHIFT) : (int)(ent >> FC_SHIFT);
                    float4 v;
                    if (BIG) {
                        const int tg = (int)(ent & (FC_BIGT - 1));
                        // (exact: the quotients stay below 2^13 and the fractions at least 1 / (2 s) from an integer)
                        const int q = (int)(((float)tg + 0.5f) * inv_s3), i3 = tg - q * bx.s3;
                        const int i1 = (int)(((float)q + 0.5f) * inv_s2), i2 = q - i1 * bx.s2;
                        const float n1 = (float)(i1 - bx.R1), n2 = (float)(i2 - bx.R2), n3 = (float)(i3 - bx.R3);
                        v.x = fmaf(L.t[6], n3, fmaf(L.t[3], n2, L.t[0] * n1));      // as build_shift_table makes them
                        v.y = fmaf(L.t[7], n3, fmaf(L.t[4], n2, L.t[1] * n1));
                        v.z = fmaf(L.t[8], n3, fmaf(L.t[5], n2, L.t[2] * n1));
                        v.w = 0.0f;
                    } else {
                        v = tab[ent & (FC_TCAP - 1)];
                    }
                    const float4 pa = pairA[pp];
                    const float dx = pa.x + v.x, dy = pa.y + v.y, dz = pa.z + v.z;
                    const float d2 = fmaf(dx, dx, fmaf(dy, dy, dz * dz));
                    const float w = hw_exp2(a2 * (d2 - pa.w)) * pairC[pp];
                    {
                        const float d = hw_sqrt(d2);
                        const float u = d * bc.inv_interval;
                        int start = (int)(u - bc.start_off);          // truncation toward zero
                        start = max(0, min(start, NBINS - WLr));
                        const float beta_c = ((float)(start + WLr / 2 + 1) - u) * bc.len_step;
                        const WindowSeed s = window_seed(beta_c, bc.len_step, w);
#ifndef CFH_EXP_NOCONFLICT
                        window_scatter_rn<WL>(hist + start, s, bc.len_cc, WLr);
#else
                        window_scatter_rn<WL>(hist + (start & 0) + lane, s, bc.len_cc, WLr);
#endif
                    }
                    if (HAS_ANG) {
                        if (d2 > 1e-5f) {       // the self image contributes to S and the distance encoding only
                            const float rinv = hw_rsq(d2);
#pragma unroll
                            for (int ax = 0; ax < 3; ax++) {
                                float cs = (dx * f[ax][0] + dy * f[ax][1] + dz * f[ax][2]) * rinv;
                                if (COS_ABS) cs = fabsf(cs);
                                const float uu = (cs - bc.ang_mu0) * bc.ang_inv_interval;      // in bin units
                                if (ANG == SMALL_A) {
                                    // all 16 basis values, outwards from bin 8 by the two-sided recurrence (sigma >= 1
                                    // bin: the value at bin 8 is at least e^-32 of the peak, no underflow)
                                    const WindowSeed sa = window_seed(((float)(SMALL_A / 2) - uu) * bc.ang_step, bc.ang_step, w);
                                    window_scatter_rn<SMALL_A>(hist + HW_DIST + (lane & (A16_COPIES - 1)) * A16_STRIDE + ax * SMALL_A,
                                                               sa, bc.ang_cc);
                                    continue;
                                }
                                const float mf = clampf(__builtin_rintf(uu), 0.0f, (float)(NBINS - 1));
                                const float eps = 2.0f * (uu - mf);
#ifndef CFH_EXP_NOCONFLICT
                                int32_t* hb = hist + HW_DIST + ax * NORD * NBINS + (int)mf;
#else
                                int32_t* hb = hist + HW_DIST + ax * NORD * NBINS + ((int)mf & 0) + lane;
#endif
                                float val = w;
                                atomicAdd(hb, rint_i(val));
#pragma unroll
                                for (int o = 1; o < NORD; o++) { val *= eps; atomicAdd(hb + o * NBINS, rint_i(val)); }
                            }
                        }
                    }
                }
            }
            n_eval += (unsigned long long)nlist;
        };
        auto heavy = [&](int nlist) { heavy_impl(nlist, std::false_type{}); };

        for (int g0 = 0; g0 < npairs; g0 += FC_GROUP) {
            const float rx = nrx, ry = nry, rz = nrz;
            const float2 k2 = nk2, v2 = nv2;
            float d2min = nnear;
            if (g0 + FC_GROUP < npairs) fetch(g0 + FC_GROUP);
            const bool active = g0 + pr < npairs;
            const float rn = hw_sqrt(fmaf(rx, rx, fmaf(ry, ry, rz * rz)));

            float Sb, S;
            int nlist;
            bool spilled;                     // (several chunks) more survivors than the list holds: the chunks again, one by one
            bool known = near_known;
            for (;;) {
            // ---- pass A: nearest image (known beforehand for the usual box)
            CFH_PH(1);
            if (!known) {
                d2min = 3.0e38f;
                sweep(active, rx, ry, rz, sorted ? fmaf(2.0002f, rn, 1e-4f) : FC_REACH_ALL,
                      [&](bool in, int, int, float d2, int cnt_in) { d2min = in ? fminf(d2min, d2) : d2min; n_seen += cnt_in; });
                d2min = half_min(d2min);
            }

            // ---- pass B: weights, normaliser and (one-chunk tables) the survivors
            CFH_PH(2);
            const float reachB = sorted ? fmaf(1.0001f, rn + hw_sqrt(d2min + cutS), 1e-4f) : FC_REACH_ALL;
            Sb = 0.0f;
            nlist = 0;
            spilled = false;
            if (nchunks == 1) {
                sweep(active, rx, ry, rz, reachB, [&](bool in, int t, int, float d2, int cnt_in) {
                    const float ex = in ? a2 * (d2 - d2min) : -INF;      // (2^-inf = 0, and -inf is below every threshold)
                    Sb += hw_exp2(ex);
                    n_seen += cnt_in;
                    const bool keep = ex >= prune;
                    const uint64_t m = ballot(keep);
                    if (keep) list[nlist + lane_prefix(m)] = (uint16_t)((pr << FC_SHIFT) | t);
                    nlist += __popcll(m);
                });
            } else {
                sweep(active, rx, ry, rz, reachB, [&](bool in, int t, int t0c, float d2, int cnt_in) {
                    const float ex = in ? a2 * (d2 - d2min) : -INF;
                    Sb += hw_exp2(ex);
                    n_seen += cnt_in;
                    if (one_list && !spilled) {
                        const bool keep = ex >= prune;
                        const uint64_t m = ballot(keep);
                        if (nlist + __popcll(m) > FC_LISTCAP) spilled = true;
                        else {
                            if (keep) list[nlist + lane_prefix(m)] = (uint16_t)((pr << FC_BIGSHIFT) | (t0c + t));
                            nlist += __popcll(m);
                        }
                    }
                });
            }
            S = half_sum(Sb);
            // a reference borrowed from the usual box may lie far above the nearest image of a larger box (a strongly
            // sheared cell): a sum of weights of 2^24 and more says so (with the nearest image as the reference it is at
            // most the number of translations, 2^13), and the group is done again with a sweep for the nearest
            if (known && !sorted && ballot(active && !(S < 0x1p24f)) != 0) { known = false; continue; }
            break;
            }

            // ---- logits, running softmax
            CFH_PH(3);
            const float qk = half_sum(fmaf(q2.x, k2.x, q2.y * k2.y));
            const float z = fmaf(hw_log2(S), LN2, a * d2min);
            const float logit = active ? qk + z : -INF;
            const float gmax = uniform_f(wave_maxf(logit));
            if (gmax > m_run) {
                if (m_run > -INF) {
                    const float fac = hw_exp2((m_run - gmax) * LOG2E);
                    if (VEC) {
                        constexpr int NW = VEC ? HWK / (4 * WAVE) : 1;
                        int4 hv[NW];
#pragma unroll
                        for (int u = 0; u < NW; u++) hv[u] = reinterpret_cast<const int4*>(hist)[lane + WAVE * u];
#pragma unroll
                        for (int u = 0; u < NW; u++)
                            reinterpret_cast<int4*>(hist)[lane + WAVE * u] =
                                make_int4(rint_i((float)hv[u].x * fac), rint_i((float)hv[u].y * fac),
                                          rint_i((float)hv[u].z * fac), rint_i((float)hv[u].w * fac));
                    } else {
                        for (int u = lane; u < HWL; u += WAVE) hist[u] = rint_i((float)hist[u] * fac);
                    }
                    accv.x *= fac; accv.y *= fac; Dl *= fac;
                }
                m_run = gmax;
            }
            const float ew = active ? hw_exp2((logit - m_run) * LOG2E) : 0.0f;
            accv.x = fmaf(ew, v2.x, accv.x);
            accv.y = fmaf(ew, v2.y, accv.y);
            if (sub == 0 && active) {
                const uint32_t eh = ((uint32_t)(e0 + g0 + pr) * (uint32_t)H + (uint32_t)h) * 4u;      // byte offset
                pairA[pr] = make_float4(rx, ry, rz, d2min);
                pairC[pr] = ew * hw_rcp(S) * fixs;
                *reinterpret_cast<float*>(reinterpret_cast<char*>(C.z) + eh) = z;
                if (npairs <= FC_LOGCAP) logit_s[g0 + pr] = logit;
                else *reinterpret_cast<float*>(reinterpret_cast<char*>(C.prob) + eh) = logit;      // the logit for now; normalised when the row is complete
                Dl += ew;
            }
            wave_sync();

            // ---- heavy pass
            CFH_PH(4);
            if (nchunks == 1) heavy(nlist);
            else if (one_list && !spilled) heavy_impl(nlist, std::true_type{});
            else {
                for (int ch = 0; ch < nchunks; ch++) {
                    const int t0c = ch * FC_TCAP;
                    const int cnt = min(FC_TCAP, bx.T - t0c);
                    wave_sync();
                    build_shift_table(tab, t0c, cnt, bx, L, lane);
                    wave_sync();
                    int nl = 0;
                    for (int t0 = 0; t0 < cnt; t0 += FC_GROUP) {
                        const int t = t0 + sub;
                        const float4 v = tab[min(t, cnt - 1)];
                        const float dx = rx + v.x, dy = ry + v.y, dz = rz + v.z;
                        const float ex = a2 * (fmaf(dx, dx, fmaf(dy, dy, dz * dz)) - d2min);
                        const bool keep = active && t < cnt && ex >= prune;
                        const uint64_t m = ballot(keep);
                        if (keep) list[nl + lane_prefix(m)] = (uint16_t)((pr << FC_SHIFT) | t);
                        nl += __popcll(m);
                    }
                    wave_sync();
                    heavy(nl);
                }
            }
            wave_sync();                      // list, pair data and (several chunks) the table may be rewritten
            CFH_PH(3);
        }

        // ---- the row is complete: normalise and write
        CFH_PH(7);
        const float D = uniform_f(wave_sum(Dl));
        const float inv = D > 0.0f ? hw_rcp(D) : 0.0f;
        {
            const float ox = rows8_sum(accv.x) * inv, oy = rows8_sum(accv.y) * inv;
            if (lane < FC_GROUP) *reinterpret_cast<float2*>(C.out + ih * DH + 2 * sub) = make_float2(ox, oy);
        }
        {
            // all reads first (one LDS round trip instead of one per word), then store; a lane takes four
            // consecutive words at a time
            const float sc = inv * hw_rcp(fixs);
            float* dst = C.hist + ((size_t)h * P.N + i) * HWK;      // head-major: the rows of a head are contiguous
            if (ANG == SMALL_A) {
                // distance bins as they are, every angle bin as the sum of its copies (integers: any order), zeros behind
                for (int u = lane; u < HWK; u += WAVE) {
                    int32_t sum = 0;
                    if (u < HW_DIST) sum = hist[u];
                    else if (u < HW_DIST + 3 * SMALL_A) {
#pragma unroll
                        for (int c = 0; c < A16_COPIES; c++) sum += hist[HW_DIST + c * A16_STRIDE + (u - HW_DIST)];
                    }
                    dst[u] = (float)sum * sc;
                }
            } else if (VEC) {
                constexpr int NW = VEC ? HWK / (4 * WAVE) : 1;
                int4 hv[NW];
#pragma unroll
                for (int u = 0; u < NW; u++) hv[u] = reinterpret_cast<const int4*>(hist)[lane + WAVE * u];
#pragma unroll
                for (int u = 0; u < NW; u++)
                    reinterpret_cast<float4*>(dst)[lane + WAVE * u] =
                        make_float4((float)hv[u].x * sc, (float)hv[u].y * sc, (float)hv[u].z * sc, (float)hv[u].w * sc);
            } else {
                for (int u = lane; u < HWK; u += WAVE) dst[u] = (float)hist[u] * sc;
            }
        }
        if (npairs <= FC_LOGCAP) {                               // logits -> probabilities
            for (int el = lane; el < npairs; el += WAVE)
                C.prob[(size_t)(e0 + el) * H + h] = hw_exp2((logit_s[el] - m_run) * LOG2E) * inv;
        } else {
            for (int g0 = 0; g0 < npairs; g0 += FC_GROUP) {      // each was written by the lane that now reads it
                if (sub == 0 && g0 + pr < npairs) {
                    const size_t eh = (size_t)(e0 + g0 + pr) * H + h;
                    C.prob[eh] = hw_exp2((C.prob[eh] - m_run) * LOG2E) * inv;
                }
            }
        }
        CFH_PH_FLUSH(P.stats);
        if (P.stats && lane == 0) {
            atomicAdd(P.stats + STAT_FWD_EVAL, n_eval);
            atomicAdd(P.stats + STAT_FWD_RAW, (unsigned long long)bx.T * (unsigned long long)npairs);
            atomicAdd(P.stats + STAT_FWD_PAIRS, (unsigned long long)npairs);
            atomicAdd(P.stats + STAT_FWD_SEEN, n_seen);
        }
    }
}

// out (N,H,16) += Wcat_h (16, hw) . hist (H,N,hw): one workgroup of PROJ_WAVES wavefronts per (16 atoms, head); each
// wavefront takes a slice of the reduction index through MFMA 16x16x4 (the four lanes of a row read 64 consecutive
// bytes of it per load), the slices meet in LDS and are added in a fixed order by the first
// wavefront (no atomics: the result does not depend on timing).  grid (ceil(N/16), H), block 64 * PROJ_WAVES.
constexpr int PROJ_WAVES = 4;
__global__ __launch_bounds__(WAVE * PROJ_WAVES) void core_project_kernel(const float* __restrict__ hist,
                                                                         const float* __restrict__ wcat,
                                                                         float* __restrict__ out, int N, int H, int hw) {
    __shared__ float part[PROJ_WAVES][4][WAVE];
    const int lane = threadIdx.x & (WAVE - 1), wv = threadIdx.x >> 6, col = lane & 15, kk = lane >> 4;
    const int h = blockIdx.y, i0 = blockIdx.x * 16;
    const int row = min(i0 + col, N - 1);
    // the four lanes (kk) of a row read 64 consecutive bytes per load; which word of the reduction index a lane
    // holds does not matter as long as both operands agree
    const float4* ap = reinterpret_cast<const float4*>(hist + ((size_t)h * N + row) * hw) + kk;
    const float4* bp = reinterpret_cast<const float4*>(wcat + ((size_t)h * DH + col) * hw) + kk;
    v4f_c acc = {0.f, 0.f, 0.f, 0.f};
    const int steps = hw / 64, per = (steps + PROJ_WAVES - 1) / PROJ_WAVES;
    const int s_begin = wv * per, s_end = min(steps, s_begin + per);
#pragma unroll 2
    for (int s = s_begin; s < s_end; s++) {
        float4 a4[4], b4[4];
#pragma unroll
        for (int u = 0; u < 4; u++) { a4[u] = ap[16 * s + 4 * u]; b4[u] = bp[16 * s + 4 * u]; }
#pragma unroll
        for (int u = 0; u < 4; u++) {
            acc = __builtin_amdgcn_mfma_f32_16x16x4f32(a4[u].x, b4[u].x, acc, 0, 0, 0);
            acc = __builtin_amdgcn_mfma_f32_16x16x4f32(a4[u].y, b4[u].y, acc, 0, 0, 0);
            acc = __builtin_amdgcn_mfma_f32_16x16x4f32(a4[u].z, b4[u].z, acc, 0, 0, 0);
            acc = __builtin_amdgcn_mfma_f32_16x16x4f32(a4[u].w, b4[u].w, acc, 0, 0, 0);
        }
    }
#pragma unroll
    for (int r = 0; r < 4; r++) part[wv][r][lane] = acc[r];
    __syncthreads();
    if (wv != 0) return;
    // component r of lane (kk, col): atom 4 kk + r of the tile, channel col
#pragma unroll
    for (int r = 0; r < 4; r++) {
        float sum = part[0][r][lane];
#pragma unroll
        for (int w = 1; w < PROJ_WAVES; w++) sum += part[w][r][lane];
        const int it = i0 + 4 * kk + r;
        if (it < N) out[((size_t)it * H + h) * DH + col] += sum;
    }
}

// G (H,N,hw) = go (N,H,16) . Wcat_h (16, hw): wavefront per (16 atoms, head, 64-word block); four MFMA tiles whose
// columns are interleaved (tile t, column c <-> word 4 c + t) so that a lane stores 16 consecutive bytes.
// grid (ceil(N/16), H, hw/64).  `queues`: optional work-queue heads to clear (when no prepare launch does).
// Records kept from the forward pass (`slow.items` not null): the wavefronts (x, 0, 0) with x a multiple of
// SLOW_GB_BLOCKS also list the records of SLOW_GB_BLOCKS x 16 atoms whose box is not the usual one, for the main kernel of the backward pass to take first (as prepare_items_block does for the forward,
// whose lists are gone by now).
constexpr int SLOW_GB_BLOCKS = 4;
struct SlowListArgs {
    uint32_t* items;       // (N, H, REC_WORDS) or null
    int32_t* count;        // (lists), lists = ceil(ceil(N / 16) / SLOW_GB_BLOCKS)
    int32_t* list;         // (lists, SLOW_GB_BLOCKS x 16 x H)
    int32_t R;             // half-width of the usual box
};
__global__ __launch_bounds__(WAVE) void core_gbuild_kernel(const float* __restrict__ go, const float* __restrict__ wcat,
                                                           float* __restrict__ G, int N, int H, int hw,
                                                           int32_t* __restrict__ queues, const SlowListArgs slow) {
    const int lane = threadIdx.x, col = lane & 15, kk = lane >> 4;
    const int h = blockIdx.y, i0 = blockIdx.x * 16;
    if (queues && blockIdx.x == 0 && blockIdx.y == 0 && blockIdx.z == 0)      // work queues of the launch that follows
        for (int u = lane; u < H * NQUEUE; u += WAVE) queues[u * QSTRIDE] = 0;
    if (slow.items && blockIdx.y == 0 && blockIdx.z == 0 && blockIdx.x % SLOW_GB_BLOCKS == 0) {
        const int li = (int)blockIdx.x / SLOW_GB_BLOCKS;
        const int first = (int)blockIdx.x * 16 * H, last = min(first + SLOW_GB_BLOCKS * 16 * H, N * H);
        const uint32_t usual = (uint32_t)(slow.R | (slow.R << 8) | (slow.R << 16));
        int listed = 0;
        for (int r0 = first; r0 < last; r0 += 4 * WAVE) {
            // (four loads that do not wait for each other, then their ranks)
            uint32_t boxw[4];
#pragma unroll
            for (int u = 0; u < 4; u++) {
                const int r = r0 + u * WAVE + lane;
                boxw[u] = r < last ? slow.items[(size_t)r * REC_WORDS + REC_BOX] : usual;
            }
#pragma unroll
            for (int u = 0; u < 4; u++) {
                const int r = r0 + u * WAVE + lane;
                const bool own = r < last && (boxw[u] & 0x00ffffffu) != usual;
                const uint64_t m = ballot(own);
                const int rank = listed + __popcll(m & ((1ull << lane) - 1ull));
                if (r < last) {
                    if (own) slow.list[(size_t)li * (SLOW_GB_BLOCKS * 16 * H) + rank] = r;
                    const uint32_t neww = own ? (boxw[u] | REC_BOX_LISTED_BWD) : (boxw[u] & ~REC_BOX_LISTED_BWD);
                    if (neww != boxw[u]) slow.items[(size_t)r * REC_WORDS + REC_BOX] = neww;
                }
                listed += __popcll(m);
            }
        }
        if (lane == 0) slow.count[li] = listed;
    }
    const int row = min(i0 + col, N - 1);
    const float4 a4 = reinterpret_cast<const float4*>(go + ((size_t)row * H + h) * DH)[kk];      // channels 4 kk ..
    const float A[4] = {a4.x, a4.y, a4.z, a4.w};
    {
        const int w0 = blockIdx.z * 64;
        float4 b4[4];
#pragma unroll
        for (int j = 0; j < 4; j++)
            b4[j] = *reinterpret_cast<const float4*>(wcat + ((size_t)h * DH + 4 * kk + j) * hw + w0 + 4 * col);
        v4f_c acc[4];
#pragma unroll
        for (int t = 0; t < 4; t++) acc[t] = v4f_c{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int j = 0; j < 4; j++) {
            acc[0] = __builtin_amdgcn_mfma_f32_16x16x4f32(A[j], b4[j].x, acc[0], 0, 0, 0);
            acc[1] = __builtin_amdgcn_mfma_f32_16x16x4f32(A[j], b4[j].y, acc[1], 0, 0, 0);
            acc[2] = __builtin_amdgcn_mfma_f32_16x16x4f32(A[j], b4[j].z, acc[2], 0, 0, 0);
            acc[3] = __builtin_amdgcn_mfma_f32_16x16x4f32(A[j], b4[j].w, acc[3], 0, 0, 0);
        }
#pragma unroll
        for (int r = 0; r < 4; r++) {
            const int it = i0 + 4 * kk + r;
            if (it < N)
                *reinterpret_cast<float4*>(G + ((size_t)h * N + it) * hw + w0 + 4 * col) =
                    make_float4(acc[0][r], acc[1][r], acc[2][r], acc[3][r]);
        }
    }
}

// gwcat (slice,H,16,hw) = sum over a slice of the atoms of go (.,h,16) (x) hist (h,.,hw): wavefront per (head, 64-word
// block, slice); four MFMA tiles with interleaved columns as above.  grid (ceil(hw/64 / GW_WPB), H, nslices), at most
// CORE_GW_SLICES slices.
__device__ __forceinline__ void core_gwcat_block(const float* __restrict__ go, const float* __restrict__ hist,
                                                 float* __restrict__ gwcat, int N, int H, int hw, int per_slice, int slice) {
    // the GW_WPB wavefronts of a workgroup take neighbouring pieces of the same rows at the same time: GW_WPB x 256
    // contiguous bytes of a row instead of 256 bytes every 4 KB (82 -> 70 us for the four layers of the benchmark)
    const int lane = threadIdx.x & (WAVE - 1), col = lane & 15, kk = lane >> 4;
    const int w0 = ((int)blockIdx.x * (int)(blockDim.x >> 6) + (int)(threadIdx.x >> 6)) * 64, h = blockIdx.y;
    if (w0 >= hw) return;
    const int i_begin = slice * per_slice, i_end = min(N, i_begin + per_slice);
    v4f_c acc[4];
#pragma unroll
    for (int t = 0; t < 4; t++) acc[t] = v4f_c{0.f, 0.f, 0.f, 0.f};
    // GW_DEPTH x 16 atoms per step, all their loads asked for before the first product: a wavefront keeps 16 KB of
    // histogram rows in flight (with 4 KB the kernel ran at 40 % of the bandwidth it reaches now)
    constexpr int GW_DEPTH = 4;
    for (int ib = i_begin; ib < i_end; ib += 16 * GW_DEPTH) {
        float av[GW_DEPTH][4];
        float4 bv[GW_DEPTH][4];
#pragma unroll
        for (int d = 0; d < GW_DEPTH; d++)
#pragma unroll
            for (int j = 0; j < 4; j++) {
                // (no branch around the loads: an atom past the end reads the slice's first one, with go as zero)
                const int it = ib + 16 * d + 4 * j + kk;
                const bool live = it < i_end;
                const int itc = live ? it : i_begin;
                const float g = go[((size_t)itc * H + h) * DH + col];
                av[d][j] = live ? g : 0.0f;
                bv[d][j] = *reinterpret_cast<const float4*>(hist + ((size_t)h * N + itc) * hw + w0 + 4 * col);
            }
        // (without the branches the compiler would put every load next to its product: 113 us instead of 78)
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int d = 0; d < GW_DEPTH; d++)
#pragma unroll
            for (int j = 0; j < 4; j++) {
                acc[0] = __builtin_amdgcn_mfma_f32_16x16x4f32(av[d][j], bv[d][j].x, acc[0], 0, 0, 0);
                acc[1] = __builtin_amdgcn_mfma_f32_16x16x4f32(av[d][j], bv[d][j].y, acc[1], 0, 0, 0);
                acc[2] = __builtin_amdgcn_mfma_f32_16x16x4f32(av[d][j], bv[d][j].z, acc[2], 0, 0, 0);
                acc[3] = __builtin_amdgcn_mfma_f32_16x16x4f32(av[d][j], bv[d][j].w, acc[3], 0, 0, 0);
            }
    }
    // component r of tile t, lane (kk, col): channel 4 kk + r, word w0 + 4 col + t.  Every slice writes its own
    // copy (slice, H, 16, hw) in full: nothing to clear, no atomics, and the sum over the slices that follows is made
    // in a fixed order
    float* const part = gwcat + (size_t)slice * H * DH * hw;
#pragma unroll
    for (int r = 0; r < 4; r++)
        *reinterpret_cast<float4*>(part + ((size_t)h * DH + 4 * kk + r) * hw + w0 + 4 * col) =
            make_float4(acc[0][r], acc[1][r], acc[2][r], acc[3][r]);
}
constexpr int GW_WPB = 4;          // wavefronts per workgroup of the two kernels below (8: the same; 16: far slower)
__global__ __launch_bounds__(WAVE * GW_WPB) void core_gwcat_kernel(const float* __restrict__ go, const float* __restrict__ hist,
                                                          float* __restrict__ gwcat, int N, int H, int hw, int per_slice) {
    core_gwcat_block(go, hist, gwcat, N, H, hw, per_slice, (int)blockIdx.z);
}
// several jobs: grid (ceil(hw/64 / GW_WPB), H, slices of all jobs); the job of a slice by a scan of the (few) jobs
__global__ __launch_bounds__(WAVE * GW_WPB) void core_gwcat_multi_kernel(const CoreWgradJobs T) {
    int j = 0;
    while (j + 1 < T.njobs && (int)blockIdx.z >= T.job[j + 1].slice0) j++;
    const CoreWgradJob& J = T.job[j];
    core_gwcat_block(J.go, J.hist, J.gwcat, J.N, T.H, T.hw, J.per_slice, (int)blockIdx.z - J.slice0);
}
// grid (H*16, jobs): added to the destinations
__global__ __launch_bounds__(256) void core_gw_finish_multi_kernel(const CoreWgradJobs T) {
    const CoreWgradJob& J = T.job[blockIdx.y];
    core_gw_finish_block<true>(J.gwcat, J.nslices, (size_t)T.H * DH * T.hw, T.hw, T.dist_coef, T.angle_coef, T.ws,
                               J.gW[0], J.gW[1], J.gW[2], J.gW[3], (int)blockIdx.x);
}


// =================================================================================================================
// backward
// =================================================================================================================
// Per item: G = Wcat^T go (made by core_gbuild_kernel) in LDS; for every image n of pair j with probability
// p_n = exp(a d^2 - z) the value bg_n = sum_k b_k(d_n) G_k + sum_axis sum_o eps^o G'_(axis,o,m*) is gathered, and
//     go . psi_ij          = sum_n p_n bg_n                                   (per pair, fixed-point LDS sums)
//     gl_ij = dL/dlogit_ij = P_ij (go . v_j + go . psi_ij - go . out_i)
//     ga_ih                = sum_j P_ij [(go . v_j - go . out_i) A0_j + sum_n p_n d_n^2 bg_n],  A0_j = sum_n p_n d_n^2
//     gq_i                 = sum_j gl_ij k_j
// (the terms A0_j (go . psi_ij) of dL/dz and of the covariance form cancel).  gk and gv are sums over the pairs that
// point AT an atom and are left to the column kernel of the attention backward (from gl and P).
template <int HWK>
struct CoreBwdShared {
    float4 tab[FC_TCAP];
    uint16_t list[FC_LISTCAP];
    float Gs[HWK];
    float4 pairA[FC_GROUP];      // rx, ry, rz, z log2(e)
    float pairP[FC_GROUP];       // P_ij
    int32_t pairB[FC_GROUP];     // sum_n P_ij p_n bg_n in fixed point
};
template <int WL, int ANG, bool COS_ABS>
__global__ __launch_bounds__(WAVE * CORE_WPB) void fused_core_bwd_kernel(const CoreArgs C) {
    constexpr bool HAS_ANG = ANG > 0;
    constexpr int HWK = core_hist_words(ANG);
    __shared__ CoreBwdShared<HWK> shared[CORE_WPB];
    CoreBwdShared<HWK>& sh = shared[threadIdx.x >> 6];
    float4* const tab = sh.tab;
    uint16_t* const list = sh.list;
    float* const Gs = sh.Gs;
    float4* const pairA = sh.pairA;
    float* const pairP = sh.pairP;
    int32_t* const pairB = sh.pairB;

    const KernelArgs& P = C.K;
    const int lane = threadIdx.x & (WAVE - 1);
    const int H = P.H;
    const int wid = core_wave_record(C, (int)blockIdx.x * CORE_WPB + (int)(threadIdx.x >> 6), lane);
    if (wid < 0) return;
    const int it_cur = div_heads(P, wid);      // one wavefront per item, long items first
    const int h = wid - it_cur * H;
    const int pr = lane >> 3, sub = lane & 7;
    const BasisConsts bc = P.bc;
    const int WLr = WL > 0 ? WL : bc.len_window;      // bins of the distance window (WL == 0: known at run time only)
    const float prune = (P.prune_log2 > 0.0f) ? -P.prune_log2 : -3.0e38f;
    const float INF = __builtin_inff();

    if (it_cur >= P.N) return;
    {
        const uint32_t rec_cur = load_record_lane(P, it_cur, h, lane);
        if (core_record_taken_elsewhere(C, rec_cur, wid, lane)) return;
        const CoreItem ci = core_unpack(C, rec_cur, true);
        const int i = ci.item.i;
        const float a2 = ci.item.a * LOG2E;
        const Lattice L = ci.item.L;
        const Box bx = ci.item.bx;
        const bool sorted = ci.sorted;
        const int nchunks = ci.nchunks;
        float f[3][3];
        if (HAS_ANG) {
#pragma unroll
            for (int ax = 0; ax < 3; ax++)
#pragma unroll
                for (int d = 0; d < 3; d++) f[ax][d] = rec_f(rec_cur, REC_FRAMES + ax * 3 + d);
        }
        const int e0 = ci.item.e0, npairs = ci.item.npairs;
        const size_t ih = (size_t)i * H + h;
        core_load_table(C, ci, tab, lane);
        float gabs = 0.0f;
        {
            const float* src = C.G + ((size_t)h * P.N + i) * HWK;
            if (HWK >= 4 * WAVE) {
                constexpr int NW = HWK >= 4 * WAVE ? HWK / (4 * WAVE) : 1;
                float4 g4[NW];
#pragma unroll
                for (int u = 0; u < NW; u++) g4[u] = reinterpret_cast<const float4*>(src)[lane + WAVE * u];
#pragma unroll
                for (int u = 0; u < NW; u++) {
                    reinterpret_cast<float4*>(Gs)[lane + WAVE * u] = g4[u];
                    gabs += (fabsf(g4[u].x) + fabsf(g4[u].y)) + (fabsf(g4[u].z) + fabsf(g4[u].w));
                }
            } else {
                for (int u = lane; u < HWK; u += WAVE) { const float g = src[u]; Gs[u] = g; gabs += fabsf(g); }
            }
        }
        const float2 go2 = *reinterpret_cast<const float2*>(C.go + ih * DH + 2 * sub);
        const float2 ov2 = *reinterpret_cast<const float2*>(C.outv + ih * DH + 2 * sub);
        const float c0 = half_sum(fmaf(go2.x, ov2.x, go2.y * ov2.y));          // go . out_i
        const float gnorm = uniform_f(wave_sum(gabs));                          // |bg| <= sum |G|
        const float inv_a2 = a2 < 0.0f ? hw_rcp(a2) : 0.0f;             // (for a bound with margins)
        const float bscale = 1073741824.0f / fmaxf(gnorm, 1e-20f);      // (finite: 2^30 / 1e-30 would not be)
        const float binv = fmaxf(gnorm, 1e-20f) * (1.0f / 1073741824.0f);
        wave_sync();
        float cov = 0.0f;
        float2 gq2 = make_float2(0.f, 0.f);
        unsigned long long n_eval = 0;

        float nrx = 0.f, nry = 0.f, nrz = 0.f, nz = 0.f, npb = 0.f;
        float2 nk2 = make_float2(0.f, 0.f), nv2 = nk2;
        auto fetch = [&](int g0) {
            // (no branch per row: a row past the end re-reads the row's last pair; nothing of it is used)
            const uint32_t el = (uint32_t)min(g0 + pr, npairs - 1);
            const uint32_t e = min((uint32_t)e0 + el, (uint32_t)(P.E - 1));
            const uint32_t jh = ((((uint32_t)ci.j0 + el) * (uint32_t)H + (uint32_t)h) * DH + 2u * sub) * 4u;
            const uint32_t eh = (e * (uint32_t)H + (uint32_t)h) * 4u;
            const float3 r3 = load_at<float3>(P.rpos, e * 12u);
            nrx = r3.x; nry = r3.y; nrz = r3.z;
            nz = load_at<float>(C.z, eh); npb = load_at<float>(C.prob, eh);
            nk2 = load_at<float2>(C.k, jh);
            nv2 = load_at<float2>(C.v, jh);
        };
        if (npairs > 0) fetch(0);

        // several chunks: the survivors of all chunks in one list with their index in the whole box (as in the forward)
        const bool one_list = nchunks > 1 && bx.T <= FC_BIGT;
        auto heavy_impl = [&](int nlist, auto big) {
            constexpr bool BIG = decltype(big)::value;      // entries (pair << FC_BIGSHIFT | index in the box), no table
            // (hardware reciprocals, within an ulp: the quotients below stay exact all the same)
            const float inv_s3 = BIG ? hw_rcp((float)bx.s3) : 0.0f, inv_s2 = BIG ? hw_rcp((float)bx.s2) : 0.0f;
            for (int base = 0; base < nlist; base += WAVE) {
                const int idx = base + lane;
                if (idx < nlist) {
                    const uint32_t ent = list[idx];
                    const int pp = BIG ? (int)(ent >> FC_BIGSHIFT) : (int)(ent >> FC_SHIFT);
                    float4 v;
                    if (BIG) {
                        const int tg = (int)(ent & (FC_BIGT - 1));
                        // (exact: the quotients stay below 2^13 and the fractions at least 1 / (2 s) from an integer)
                        const int q = (int)(((float)tg + 0.5f) * inv_s3), i3 = tg - q * bx.s3;
                        const int i1 = (int)(((float)q + 0.5f) * inv_s2), i2 = q - i1 * bx.s2;
                        const float n1 = (float)(i1 - bx.R1), n2 = (float)(i2 - bx.R2), n3 = (float)(i3 - bx.R3);
                        v.x = fmaf(L.t[6], n3, fmaf(L.t[3], n2, L.t[0] * n1));      // as build_shift_table makes them
                        v.y = fmaf(L.t[7], n3, fmaf(L.t[4], n2, L.t[1] * n1));
                        v.z = fmaf(L.t[8], n3, fmaf(L.t[5], n2, L.t[2] * n1));
                        v.w = 0.0f;
                    } else {
                        v = tab[ent & (FC_TCAP - 1)];
                    }
                    const float4 pa = pairA[pp];
                    const float dx = pa.x + v.x, dy = pa.y + v.y, dz = pa.z + v.z;
                    const float d2 = fmaf(dx, dx, fmaf(dy, dy, dz * dz));
                    const float om = hw_exp2(fmaf(a2, d2, -pa.w)) * pairP[pp];       // P_ij p_n
                    float bg;
                    {
                        const float d = hw_sqrt(d2);
                        const float u = d * bc.inv_interval;
                        int start = (int)(u - bc.start_off);
                        start = max(0, min(start, NBINS - WLr));
                        const float beta_c = ((float)(start + WLr / 2 + 1) - u) * bc.len_step;
                        const WindowSeed s = window_seed(beta_c, bc.len_step, 1.0f);
                        bg = window_gather<WL>(Gs + start, s, bc.len_cc, WLr);
                    }
                    if (HAS_ANG) {
                        if (d2 > 1e-5f) {
                            const float rinv = hw_rsq(d2);
#pragma unroll
                            for (int ax = 0; ax < 3; ax++) {
                                float cs = (dx * f[ax][0] + dy * f[ax][1] + dz * f[ax][2]) * rinv;
                                if (COS_ABS) cs = fabsf(cs);
                                const float uu = (cs - bc.ang_mu0) * bc.ang_inv_interval;
                                if (ANG == SMALL_A) {
                                    const WindowSeed sa = window_seed(((float)(SMALL_A / 2) - uu) * bc.ang_step, bc.ang_step, 1.0f);
                                    bg += window_gather<SMALL_A>(Gs + HW_DIST + ax * SMALL_A, sa, bc.ang_cc);
                                    continue;
                                }
                                const float mf = clampf(__builtin_rintf(uu), 0.0f, (float)(NBINS - 1));
                                const float eps = 2.0f * (uu - mf);
                                const float* gb = Gs + HW_DIST + ax * NORD * NBINS + (int)mf;
                                float pw = eps, part = gb[0];
#pragma unroll
                                for (int o = 1; o < NORD; o++) { part = fmaf(pw, gb[o * NBINS], part); pw *= eps; }
                                bg += part;
                            }
                        }
                    }
                    const float ob = om * bg;
                    cov = fmaf(ob, d2, cov);
                    atomicAdd(pairB + pp, rint_i(ob * bscale));
                }
            }
            n_eval += (unsigned long long)nlist;
        };
        auto heavy = [&](int nlist) { heavy_impl(nlist, std::false_type{}); };

        for (int g0 = 0; g0 < npairs; g0 += FC_GROUP) {
            const float rx = nrx, ry = nry, rz = nrz;
            const float z2 = nz * LOG2E, pij = npb;
            const float2 k2 = nk2, v2 = nv2;
            if (g0 + FC_GROUP < npairs) fetch(g0 + FC_GROUP);
            const bool active = g0 + pr < npairs;
            const float rn = hw_sqrt(fmaf(rx, rx, fmaf(ry, ry, rz * rz)));
            // images with a d^2 log2 e - z2 >= -skip: d^2 <= (z2 - skip) / (a log2 e)
            const float dmax2 = (C.skip_log2 > 0.0f && a2 < 0.0f) ? fmaxf((z2 - C.skip_log2) * inv_a2, 0.0f) : INF;
            const float reach = sorted ? fmaf(1.0001f, rn + hw_sqrt(dmax2), 1e-4f) : FC_REACH_ALL;
            const float lim = active ? fminf(reach, FC_REACH_ALL) : -1.0f;      // (lengths are >= 0; padding: +inf)
            if (lane < FC_GROUP) pairB[lane] = 0;
            if (sub == 0 && active) {
                pairA[pr] = make_float4(rx, ry, rz, z2);
                pairP[pr] = pij;
            }
            float Ap = 0.0f;
            int nlist = 0;
            bool spilled = false;             // (several chunks) more survivors than the list holds: the chunks again, one by one
            if (nchunks == 1) {
                const int cnt = bx.T;
                for (int t0 = 0; t0 < cnt; t0 += FC_GROUP) {
                    const int t = t0 + sub;
                    const float4 v = tab[t];
                    const bool in = v.w <= lim;
                    if (sorted && ballot(in) == 0) break;
                    const float dx = rx + v.x, dy = ry + v.y, dz = rz + v.z;
                    const float d2 = fmaf(dx, dx, fmaf(dy, dy, dz * dz));
                    const float ex = in ? fmaf(a2, d2, -z2) : -INF;      // (2^-inf = 0, and -inf is below every threshold)
                    Ap = fmaf(hw_exp2(ex), d2, Ap);
                    const bool keep = ex >= prune;
                    const uint64_t m = ballot(keep);
                    if (keep) list[nlist + lane_prefix(m)] = (uint16_t)((pr << FC_SHIFT) | t);
                    nlist += __popcll(m);
                }
            } else {
                for (int ch = 0; ch < nchunks; ch++) {
                    const int t0c = ch * FC_TCAP;
                    const int cnt = min(FC_TCAP, bx.T - t0c);
                    wave_sync();
                    build_shift_table_padded(tab, t0c, cnt, bx, L, lane);
                    wave_sync();
                    for (int t0 = 0; t0 < cnt; t0 += FC_GROUP) {
                        const int t = t0 + sub;
                        const float4 v = tab[t];
                        const bool in = v.w <= lim;
                        const float dx = rx + v.x, dy = ry + v.y, dz = rz + v.z;
                        const float d2 = fmaf(dx, dx, fmaf(dy, dy, dz * dz));
                        const float ex = in ? fmaf(a2, d2, -z2) : -INF;
                        Ap = fmaf(hw_exp2(ex), d2, Ap);
                        if (one_list && !spilled) {
                            const bool keep = ex >= prune;
                            const uint64_t m = ballot(keep);
                            if (nlist + __popcll(m) > FC_LISTCAP) spilled = true;
                            else {
                                if (keep) list[nlist + lane_prefix(m)] = (uint16_t)((pr << FC_BIGSHIFT) | (t0c + t));
                                nlist += __popcll(m);
                            }
                        }
                    }
                }
            }
            const float A0 = half_sum(Ap);
            wave_sync();
            if (nchunks == 1) heavy(nlist);
            else if (one_list && !spilled) heavy_impl(nlist, std::true_type{});
            else {
                for (int ch = 0; ch < nchunks; ch++) {
                    const int t0c = ch * FC_TCAP;
                    const int cnt = min(FC_TCAP, bx.T - t0c);
                    wave_sync();
                    build_shift_table(tab, t0c, cnt, bx, L, lane);
                    wave_sync();
                    int nl = 0;
                    for (int t0 = 0; t0 < cnt; t0 += FC_GROUP) {
                        const int t = t0 + sub;
                        const float4 v = tab[min(t, cnt - 1)];
                        const float dx = rx + v.x, dy = ry + v.y, dz = rz + v.z;
                        const float ex = fmaf(a2, fmaf(dx, dx, fmaf(dy, dy, dz * dz)), -z2);
                        const bool keep = active && t < cnt && ex >= prune;
                        const uint64_t m = ballot(keep);
                        if (keep) list[nl + lane_prefix(m)] = (uint16_t)((pr << FC_SHIFT) | t);
                        nl += __popcll(m);
                    }
                    wave_sync();
                    heavy(nl);
                }
            }
            wave_sync();
            const float gov = half_sum(fmaf(go2.x, v2.x, go2.y * v2.y));          // go . v_j
            const float B1 = (float)pairB[pr] * binv;                             // P_ij (go . psi_ij)
            const float gl = active ? fmaf(pij, gov - c0, B1) : 0.0f;
            gq2.x = fmaf(gl, k2.x, gq2.x);
            gq2.y = fmaf(gl, k2.y, gq2.y);
            if (sub == 0 && active) {
                *reinterpret_cast<float*>(reinterpret_cast<char*>(C.glogit) + ((uint32_t)(e0 + g0 + pr) * (uint32_t)H + (uint32_t)h) * 4u) = gl;
                cov = fmaf(pij * (gov - c0), A0, cov);
            }
            wave_sync();                      // pair data, sums and list may be rewritten
        }
        cov = wave_sum(cov);
        {
            const float gx = rows8_sum(gq2.x), gy = rows8_sum(gq2.y);
            if (lane < FC_GROUP) *reinterpret_cast<float2*>(C.gq + ih * DH + 2 * sub) = make_float2(gx, gy);
        }
        if (lane == 0) P.out_ga[ih] = cov;
        if (P.stats && lane == 0) {
            atomicAdd(P.stats + STAT_BWD_EVAL, n_eval);
            atomicAdd(P.stats + STAT_BWD_RAW, (unsigned long long)bx.T * (unsigned long long)npairs);
            atomicAdd(P.stats + STAT_BWD_PAIRS, (unsigned long long)npairs);
        }
    }
}

}  // namespace cfh
