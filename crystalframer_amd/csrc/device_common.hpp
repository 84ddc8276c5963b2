// Device-side building blocks shared by the lattice-sum kernels (gfx950, wave64).
//
// Execution model used by every kernel in this directory:
//   * a workgroup is ONE 64-lane wavefront that owns one attention head h (= blockIdx.x % H, so
//     all wavefronts of a head land on the same XCD and share its L2 copy of that head's weights);
//   * wavefronts are persistent: each pops (atom i) work items of its head from one of the head's
//     queues in global memory until all are empty -- an exit every wavefront reaches;
//   * what an item needs (box, lattice, frame axes ...) comes as one 128-byte record written by
//     prepare_items_kernel and fetched one item ahead;
//   * for an item (i,h) the integer translations n of the box [-R1,R1]x[-R2,R2]x[-R3,R3] are
//     expanded once into an LDS table of Cartesian shifts n.L (a chunk at a time for large boxes);
//     pairs (i,j) are then processed four at a time, one per 16-lane row, lanes over translations.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace cfh {

constexpr int WAVE = 64;
constexpr int TCAP = 256;      // frame search: translations per chunk (4 KB of float4 when staged in LDS)
constexpr int NBINS = 64;      // distance bins K and angle bins A the kernels are compiled for
constexpr int DH = 16;         // head dimension the kernels are compiled for
constexpr int HS = 72;         // padded row stride (floats) of the 4 x 64 histograms in LDS
constexpr int RMAX = 32;       // safety clamp of a box half-width
constexpr float LOG2E = 1.4426950408889634f;
constexpr float SQRT_LOG2E = 1.2011224087864498f;
constexpr float LN2 = 0.6931471805599453f;

// ---- hardware transcendental units (quarter rate, ~1 ulp) -------------------------------------
__device__ __forceinline__ float hw_exp2(float x) { return __builtin_amdgcn_exp2f(x); }
__device__ __forceinline__ float hw_log2(float x) { return __builtin_amdgcn_logf(x); }
__device__ __forceinline__ float hw_rsq(float x) { return __builtin_amdgcn_rsqf(x); }
__device__ __forceinline__ float hw_rcp(float x) { return __builtin_amdgcn_rcpf(x); }
__device__ __forceinline__ float hw_sqrt(float x) { return __builtin_amdgcn_sqrtf(x); }
__device__ __forceinline__ float clampf(float x, float lo, float hi) { return fminf(fmaxf(x, lo), hi); }

// ---- reductions over a 16-lane row in DPP (VALU latency only; every lane must be active) --------
// quad_perm [1,0,3,2], quad_perm [2,3,0,1], row_half_mirror, row_mirror: after the four steps all
// 16 lanes of the row hold the reduction of the row.
template <int CTRL>
__device__ __forceinline__ float dpp_move(float x) {
    return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(x), CTRL, 0xf, 0xf, false));
}
__device__ __forceinline__ float row_min(float x) {
    x = fminf(x, dpp_move<0xB1>(x));
    x = fminf(x, dpp_move<0x4E>(x));
    x = fminf(x, dpp_move<0x141>(x));
    x = fminf(x, dpp_move<0x140>(x));
    return x;
}
__device__ __forceinline__ float row_sum(float x) {
    x += dpp_move<0xB1>(x);
    x += dpp_move<0x4E>(x);
    x += dpp_move<0x141>(x);
    x += dpp_move<0x140>(x);
    return x;
}

// ---- compaction of flagged translations into the survivor list ------------------------------------
// Lane (slot, tl) flags in `bits` which of its translations tl + 16 k (k = 0..7) of pair `slot` of the
// round survive.  The flagged ones of the whole wavefront get consecutive positions (rows in order,
// lanes of a row in order, a lane's own in ascending k): position - skip is where the entry goes in
// list[nlist ...), entries before `skip` (already processed) or beyond `room` are left out.  One row
// scan in DPP, four lane reads and a short loop over the largest number of flags of any lane replace
// a ballot / prefix / branch per k.  `code` = pair-in-group << shift | tl.  Returns the number of
// flagged entries of the wavefront.
// The lanes for which p holds, as a mask.  (HIP's __ballot takes an int: the condition is first made into 0 / 1 in a
// vector register and then compared with zero again, two vector instructions that this form does not need.)
__device__ __forceinline__ uint64_t ballot(bool p) { return __builtin_amdgcn_ballot_w64(p); }
template <int CTRL>
__device__ __forceinline__ int dpp_movei(int x) { return __builtin_amdgcn_update_dpp(0, x, CTRL, 0xf, 0xf, false); }
__device__ __forceinline__ int append_flagged(uint16_t* list, int nlist, int room, int skip, uint32_t bits,
                                              int slot, uint32_t code) {
    const int own = __popc(bits);
    int x = own;                                  // inclusive prefix within the 16-lane row (row_shr 1, 2, 4, 8)
    x += dpp_movei<0x111>(x);
    x += dpp_movei<0x112>(x);
    x += dpp_movei<0x114>(x);
    x += dpp_movei<0x118>(x);
    const int t0 = __builtin_amdgcn_readlane(x, 15), t1 = __builtin_amdgcn_readlane(x, 31);
    const int t2 = __builtin_amdgcn_readlane(x, 47), t3 = __builtin_amdgcn_readlane(x, 63);
    const int base = slot == 0 ? 0 : slot == 1 ? t0 : slot == 2 ? t0 + t1 : t0 + t1 + t2;
    int pos = base + x - own - skip;
    while (ballot(bits != 0u)) {
        if (bits != 0u) {
            const int k = __builtin_ctz(bits);
            bits &= bits - 1u;
            if (pos >= 0 && pos < room) list[nlist + pos] = (uint16_t)(code + 16u * (uint32_t)k);
            pos++;
        }
    }
    return t0 + t1 + t2 + t3;
}

// ---- reductions over the four rows of a wavefront (same column), gfx950 lane swaps ---------------
// v_permlane32_swap exchanges the upper half of one register with the lower half of another,
// v_permlane16_swap the odd rows of one with the even rows of another: applied to two copies of x
// they hand every lane the two values to combine.  VALU only, no LDS round trip.
__device__ __forceinline__ void swap32(float x, float& lo, float& hi) {
    const auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
    lo = __uint_as_float(r[0]); hi = __uint_as_float(r[1]);
}
__device__ __forceinline__ void swap16(float x, float& even, float& odd) {
    const auto r = __builtin_amdgcn_permlane16_swap(__float_as_uint(x), __float_as_uint(x), false, false);
    even = __uint_as_float(r[0]); odd = __uint_as_float(r[1]);
}
__device__ __forceinline__ float rows_sum(float x) {      // every lane: sum over lanes c, c+16, c+32, c+48
    float p, q;
    swap32(x, p, q); x = p + q;
    swap16(x, p, q); return p + q;
}
__device__ __forceinline__ float rows_min(float x) {
    float p, q;
    swap32(x, p, q); x = fminf(p, q);
    swap16(x, p, q); return fminf(p, q);
}
// ---- wave64 reductions: rows in DPP, then across the rows -----------------------------------------
__device__ __forceinline__ float wave_sum(float v) { return rows_sum(row_sum(v)); }
__device__ __forceinline__ float wave_min(float v) { return rows_min(row_min(v)); }

// Ordering point between the lanes of a ONE-wavefront workgroup that communicate through LDS.  The
// LDS executes a wavefront's instructions in order, so no hardware barrier and no wait for
// outstanding global stores is needed -- only the compiler must not move LDS accesses across.
__device__ __forceinline__ void wave_sync() {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

// slots of KernelArgs::stats
enum { STAT_FWD_EVAL = 0, STAT_FWD_RAW = 1, STAT_BWD_EVAL = 2, STAT_BWD_RAW = 3, STAT_FRAME1_RAW = 4,
       STAT_FRAME2_RAW = 5, STAT_FWD_PAIRS = 6, STAT_BWD_PAIRS = 7, STAT_FWD_SEEN = 8 };

__device__ __forceinline__ int uniform_i(int v) { return __builtin_amdgcn_readfirstlane(v); }
__device__ __forceinline__ float uniform_f(float v) {
    return __int_as_float(__builtin_amdgcn_readfirstlane(__float_as_int(v)));
}
__device__ __forceinline__ int lane_prefix(uint64_t mask) {   // set bits below this lane
    return __builtin_amdgcn_mbcnt_hi((uint32_t)(mask >> 32), __builtin_amdgcn_mbcnt_lo((uint32_t)mask, 0));
}

// ---- per-(atom, head) geometry ----------------------------------------------------------------
struct Box {
    int R1, R2, R3;   // half-widths
    int s2, s3;       // 2*R2+1, 2*R3+1
    int T;            // number of translations
    int over;         // 1: a half-width was cut back to RMAX
};

// Half-widths of the translation box.  Same operation order as the reference kernels
// (models/kernels/real_enc_frame_proj_fwd_length.cu:59-86): float32 up to (cutoff+0.01f)*rvl,
// double division by 2.0*CUDART_PI_F, ceil; no fused multiply-add.
#pragma clang fp contract(off)
__device__ __forceinline__ int half_width(float c1, float rvl, int minimum_range, int& over) {
    const float prod = c1 * rvl;
    const double v = (double)prod / (2.0 * (double)3.14159274101257324f);
    int r = (v > 0.0 && v < (double)RMAX) ? (int)ceil(v) : (v >= (double)RMAX ? RMAX : 0);
    if (v > (double)RMAX) over = 1;          // the rule asks for more than the kernels sum: reported, not silent
    if (minimum_range > 0) r = max(r, minimum_range);
    return min(r, RMAX);
}
__device__ __forceinline__ Box translation_box(float a, float rvl1, float rvl2, float rvl3,
                                               float cutoff_radius, int lattice_range,
                                               int minimum_range) {
    Box b;
    b.R1 = b.R2 = b.R3 = lattice_range;
    b.over = 0;
    if (cutoff_radius != 0.0f) {
        float cut = cutoff_radius;
        if (cut < 0.0f) cut = __fsqrt_rn(__fdiv_rn(-0.5f, a)) * (-cut);
        const float c1 = cut + 0.01f;
        b.R1 = half_width(c1, rvl1, minimum_range, b.over);
        b.R2 = half_width(c1, rvl2, minimum_range, b.over);
        b.R3 = half_width(c1, rvl3, minimum_range, b.over);
    }
    b.s2 = 2 * b.R2 + 1; b.s3 = 2 * b.R3 + 1;
    b.T = (2 * b.R1 + 1) * b.s2 * b.s3;
    return b;
}
#pragma clang fp contract(fast)

// inclusive prefix sum over the 64 lanes (row scans in DPP, row totals by lane reads)
__device__ __forceinline__ int wave_scan_incl(int x) {
    x += dpp_movei<0x111>(x);
    x += dpp_movei<0x112>(x);
    x += dpp_movei<0x114>(x);
    x += dpp_movei<0x118>(x);
    const int t0 = __builtin_amdgcn_readlane(x, 15), t1 = __builtin_amdgcn_readlane(x, 31);
    const int t2 = __builtin_amdgcn_readlane(x, 47);
    const int row = ((int)threadIdx.x & 63) >> 4;
    return x + (row == 0 ? 0 : row == 1 ? t0 : row == 2 ? t0 + t1 : t0 + t1 + t2);
}

struct Lattice { float t[9]; };   // rows = lattice vectors

// Fill tab[0..cnt) with the Cartesian shifts of translations t0..t0+cnt in the reference's loop
// order (n1 outermost, n3 innermost, ascending).
__device__ __forceinline__ void build_shift_table(float4* tab, int t0, int cnt, const Box& bx,
                                                  const Lattice& L, int lane) {
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
        v.w = 0.0f;
        tab[u] = v;
    }
}

// ---- truncated Gaussian windows by a two-sided multiplicative recurrence ------------------------
// For W equally spaced bins with scaled offsets beta_m = beta_c + (m-C)*sig (C = W/2) the values
// g_m = 2^(-beta_m^2) satisfy g_{m+1} = g_m r_m, r_{m+1} = r_m cc with cc = 2^(-2 sig^2), so a
// window costs three hardware exponentials instead of W.  The chain starts at the centre bin and
// runs outwards both ways (at most W/2 multiplications deep).  Exponents of the ratios are clamped
// so that an underflowed centre (far outside the basis range) gives zeros instead of 0*inf.
struct WindowSeed { float gc, rr, rl; };
__device__ __forceinline__ WindowSeed window_seed(float beta_c, float sig, float weight) {
    WindowSeed s;
    const float tb = 2.0f * beta_c * sig;
    const float s2 = sig * sig;
    s.gc = hw_exp2(-beta_c * beta_c) * weight;
    s.rr = hw_exp2(clampf(-(tb + s2), -100.0f, 100.0f));
    s.rl = hw_exp2(clampf(tb - s2, -100.0f, 100.0f));
    return s;
}

// Histograms are accumulated in LDS as unsigned 32-bit fixed point (FIX_ONE = 1.0), with integer
// atomics.  Measured on MI355X: a conflict-free wave64 ds_add_u32 costs about 6 LDS clocks per CU,
// a ds_add_f32 costs 190-260 whatever the addresses (the float adder takes the lanes one at a time),
// so float atomics are not usable in an inner loop.  The quantities accumulated are
// softmax-normalised weights times Gaussians, so every bin stays within [0, 1]; one unit in the last
// place is 4.7e-10, finer than a float32 accumulator.
//
// Pairs (i,j) of one (atom, head) item are processed GROUP at a time: the translations that
// survive pruning are compacted for the whole group into one LDS list (entry = pair-in-group and
// table index), and the heavy pass runs over that list 64 entries per step, so its lanes stay full
// although a single pair keeps only ~17 translations on average.  Each pair of the group has its own
// 4 x 64 histogram; a batch takes every nb-th entry of the list (nb = number of batches), so its
// lanes come from all pairs of the group, which also spreads the same-address collisions of clamped
// windows (cosines near +-1 all use the windows [0,W) or [64-W,64)).
constexpr int GROUP = 8;                           // pairs per group (forward)
constexpr int GROUP_BWD = 4;                       // pairs per group (backward: also holds G per pair)
constexpr int GROUP_BITS = 3;
constexpr int LISTCAP = 1024;                      // list entries (>= TCAP: one pair's chunk always fits)
constexpr int PAIR_STRIDE = 4 * HS + 4;            // words between the histograms of two pairs (+4 banks)
constexpr float FIX_ONE = 2147483648.0f;          // 2^31
constexpr float FIX_INV = 1.0f / 2147483648.0f;
static_assert(TCAP <= (1 << (16 - GROUP_BITS)) && GROUP <= (1 << GROUP_BITS), "list entry is 16 bits");

// Window helpers.  W > 0: the width is a compile-time constant (the loops unroll); W == 0: the width is `wrt`, the same
// in all lanes (a distance scale other than 1: any width from 2 bins to the whole basis).  The recurrence starts at
// bin C = width / 2 of the window and walks upwards to the last bin and downwards to the first.
template <int W>
__device__ __forceinline__ void window_scatter(uint32_t* base, const WindowSeed& s, float cc, int wrt = 0) {
    const int Wd = W > 0 ? W : wrt, C = Wd / 2;
    atomicAdd(base + C, (uint32_t)s.gc);
    float g = s.gc, r = s.rr;
#pragma unroll
    for (int m = C + 1; m < Wd; m++) { g *= r; r *= cc; atomicAdd(base + m, (uint32_t)g); }
    g = s.gc; r = s.rl;
#pragma unroll
    for (int m = C - 1; m >= 0; m--) { g *= r; r *= cc; atomicAdd(base + m, (uint32_t)g); }
}

// The same with the walking order chosen per lane (dir = +1: centre, upwards, then downwards; -1: centre,
// downwards, then upwards): lanes whose windows coincide (clamped windows of one pair) then add to
// different words at the same time instead of queueing on one.
template <int W>
__device__ __forceinline__ void window_scatter_dir(uint32_t* base, const WindowSeed& s, float cc, int dir, int wrt = 0) {
    const int Wd = W > 0 ? W : wrt, C = Wd / 2;
    const int up = Wd - 1 - C, down = C;            // bins above and below the centre (equal for an odd width)
    uint32_t* const centre = base + C;
    atomicAdd(centre, (uint32_t)s.gc);
    float g = s.gc, r = dir > 0 ? s.rr : s.rl;
    uint32_t* p = centre;
    const int n1 = dir > 0 ? up : down, n2 = dir > 0 ? down : up;
#pragma unroll
    for (int m = 1; m <= n1; m++) { p += dir; g *= r; r *= cc; atomicAdd(p, (uint32_t)g); }
    g = s.gc; r = dir > 0 ? s.rl : s.rr; p = centre;
#pragma unroll
    for (int m = 1; m <= n2; m++) { p -= dir; g *= r; r *= cc; atomicAdd(p, (uint32_t)g); }
}

// Scatter weight*g_m into hbase[m] and return sum_m weight*g_m*gbase[m].
template <int W>
__device__ __forceinline__ float window_scatter_gather(uint32_t* hbase, const float* gbase,
                                                       const WindowSeed& s, float cc, int wrt = 0) {
    const int Wd = W > 0 ? W : wrt, C = Wd / 2;
    float acc = s.gc * gbase[C];
    atomicAdd(hbase + C, (uint32_t)s.gc);
    float g = s.gc, r = s.rr;
#pragma unroll
    for (int m = C + 1; m < Wd; m++) { g *= r; r *= cc; acc = fmaf(g, gbase[m], acc); atomicAdd(hbase + m, (uint32_t)g); }
    g = s.gc; r = s.rl;
#pragma unroll
    for (int m = C - 1; m >= 0; m--) { g *= r; r *= cc; acc = fmaf(g, gbase[m], acc); atomicAdd(hbase + m, (uint32_t)g); }
    return acc;
}

// sum_m weight*g_m*gbase[m] alone (the histograms come from the forward pass).
template <int W>
__device__ __forceinline__ float window_gather(const float* gbase, const WindowSeed& s, float cc, int wrt = 0) {
    const int Wd = W > 0 ? W : wrt, C = Wd / 2;
    float acc = s.gc * gbase[C];
    float g = s.gc, r = s.rr;
#pragma unroll
    for (int m = C + 1; m < Wd; m++) { g *= r; r *= cc; acc = fmaf(g, gbase[m], acc); }
    g = s.gc; r = s.rl;
#pragma unroll
    for (int m = C - 1; m >= 0; m--) { g *= r; r *= cc; acc = fmaf(g, gbase[m], acc); }
    return acc;
}

// Read histogram word `idx` as a float in [0,1] and clear it.
__device__ __forceinline__ float take_bin(uint32_t* hist, int idx) {
    const uint32_t s = hist[idx];
    hist[idx] = 0u;
    return (float)s * FIX_INV;
}

// Constants of the two bases, prepared on the host.
struct BasisConsts {
    // distance basis
    float inv_interval;    // K/dist_max
    float start_off;       // 4*wscale + 1  : start = trunc(d*inv_interval - start_off)
    float len_step;        // sqrt(log2 e)/(wscale*sqrt 2) : scaled offset between neighbouring bins
    float len_cc;          // 2^(-2 len_step^2)
    int32_t len_window;    // bins of the distance window (the kernels compiled for a fixed width do not read it)
    // angle basis
    float ang_inv_interval;  // (A-1)/2 (cos_abs: A-1)
    float ang_end_off;       // 1 + 4*sigma_a
    float ang_interval;      // 2/(A-1) (cos_abs: 1/(A-1))
    float ang_sigma_inv;     // sqrt(log2 e)/(sigma_a*sqrt 2)
    float ang_step;          // ang_interval*ang_sigma_inv
    float ang_cc;            // 2^(-2 ang_step^2)
    float ang_mu0;           // centre of bin 0: -1 (cos_abs: 0)
    float ang_end_max;       // largest window end: the number of angle bins (a 16-bin basis: its 17-bin window, see basis_consts)
};

// Launch-wide arguments (by value in the kernarg segment).
struct KernelArgs {
    // geometry
    const float* a_ih; const float* rpos; const float* tvecs; const float* rvlen;
    const int64_t* batch; const int64_t* edges; const int64_t* e_start; const int32_t* order;
    // attention operands for the frame search
    const float* q; const float* k; const float* frame1;
    // value-PE operands
    const float* W[4]; const float* frames; const float* z; const float* gz; const float* gpsi;
    const float* g_pair;          // backward, optional: (E, H, 4, NBINS) the rows W^T gpsi of every pair, made by the caller
                                  // (projection weights that differ from pair to pair); the weights are then not read
    // outputs
    float* out_z; float* out_psi; float* out_d2min; float* out_frame; float* out_ga;
    float* gw_partial;            // (waves, 4, DH, NBINS) per-wave weight-gradient partials
    float* gw_out[4];             // backward: the (H, DH, NBINS) weight gradients, cleared by prepare_items_kernel
    int32_t gw_out_n;             // elements of each (0: nothing to clear)
    float* shat;                  // (E, H, 4, NBINS) window histograms: written by the forward when given,
                                  // read by the backward that does not rebuild them
    int32_t* counters;            // (H, NQUEUE) work-queue heads
    int32_t* counters2;           // optional second set, cleared along with the first: for a second kernel that
                                  // works through the same item records without a prepare launch of its own
    int32_t frames_to_records;    // frame search: also store the orthonormal frames into the item records
    int32_t contiguous_neighbours;      // the kernels of this launch take the neighbours of an atom as j0, j0 + 1, ... (the
                                        // complete n x n block per crystal, sorted by i then j): the record step checks it
    uint32_t* items;              // (N, H, REC_WORDS) item records of this launch
    int32_t* slow_count;          // optional: per block of 256 records, how many of them are listed in slow_list
    int32_t* slow_list;           // (blocks, SLOW_PREP_SLOTS) records whose box is not the usual one, for the launches that
                                  // follow to take first
    int32_t slow_R;               // half-width of the usual box
    unsigned long long* stats;    // optional running totals (see STAT_* below); never reset by a launch
    int32_t* status;              // word of the workspace header (bits, never cleared): 1 a box was cut back to RMAX;
                                  // 2 the pairs of an atom are not the consecutive neighbours j0, j0 + 1, ...
    int32_t N, E, H;
    uint32_t h_magic; int32_t h_shift;      // n / H for 0 <= n < 2^31 as (n * h_magic) >> (32 + h_shift); h_magic 0: H = 1
    float cutoff_radius; int32_t lattice_range, minimum_range;
    float prune_log2;             // <= 0: keep every translation
    float dist_coef, angle_coef, gz_coef, gw_dist_coef;
    float noise; uint32_t seed_lo, seed_hi;
    unsigned long long* seed_dev;   // optional device word mixed into the seed: prepare_items_kernel copies it
                                    // to seed_snap (what the frame search reads) and, if seed_advance, adds one
    unsigned long long* seed_snap;
    int32_t seed_advance;
    BasisConsts bc;
};

// Work distribution.  Wavefront w (= blockIdx.x) serves head w % H.  The items (atoms, visited in
// `order`: descending neighbour count, i.e. longest first) of a head are dealt round-robin to NQUEUE
// queues; a wavefront pops from queue (w / H) % NQUEUE with one global atomic per item and, when
// that queue is empty, moves to any queue of its head that is not.  Measured alternatives: ONE
// counter per head serialises its 2 400 same-address atomics (about 100 ns each) and costs more
// than the work; a static deal leaves the average wavefront idle for 40 % of the launch, and any
// wavefront that is not resident at launch doubles the makespan.
constexpr int NQUEUE = 16;
constexpr int QSTRIDE = 64;        // ints between two queue heads: each in a 256-byte block of its own
// Uniformity by construction.  The wave-level operations of the persistent loops (readfirstlane, ballot,
// DPP) must be reached by all 64 lanes together in every iteration.  The one place where a single lane
// acts for the wavefront -- the atomic that draws a ticket -- is therefore a function of its own that is
// never inlined: its lane-0 branch opens and closes inside that function, so the loop bodies that call it
// contain no branch on the lane id that an optimiser could merge with another one (a visible `lane == 0`
// test at the queue fetch and another at the stores at the end of a loop body once let the compiler thread
// the two across the back edge, and lanes 1..63 went round the loop apart from lane 0).  Everything that
// steers the loops -- the item index, "no more items" -- is a readfirstlane / ballot result, the same in
// every lane.  The price: the wait for the atomic's result sits at the end of the function instead of at
// the first use of the ticket (about a microsecond per item, hidden by the other wavefronts of the SIMD).
__device__ __attribute__((noinline)) int queue_draw(int32_t* head) {
    int v = 0;
    if (threadIdx.x == 0) v = atomicAdd(head, 1);
    return __builtin_amdgcn_readfirstlane(v);
}
__device__ __forceinline__ int queue_ticket(const KernelArgs& P, int h, int q) {
    return queue_draw(P.counters + (h * NQUEUE + q) * QSTRIDE);      // the same value in every lane
}
// Next item of head h, or -1 when every queue of the head is empty.  `q` is the queue to try first
// and is updated.
__device__ __forceinline__ int queue_pop(const KernelArgs& P, int h, int& q) {
    for (;;) {
        const int it = queue_ticket(P, h, q) * NQUEUE + q;
        if (it < P.N) return it;
        // all lanes load (lanes >= NQUEUE a copy of queue 0): no lane-dependent branch in front of the ballot
        const int ql = (int)threadIdx.x & (NQUEUE - 1);
        const int c = __hip_atomic_load(P.counters + (h * NQUEUE + ql) * QSTRIDE, __ATOMIC_RELAXED,
                                        __HIP_MEMORY_SCOPE_AGENT);
        const uint64_t m = ballot(c * NQUEUE + ql < P.N) & ((1ull << NQUEUE) - 1ull);
        if (m == 0) return -1;
        q = __builtin_ctzll(m);
    }
}
// Turns a ticket drawn earlier from queue q into an item; falls back to the other queues.
__device__ __forceinline__ int queue_redeem(const KernelArgs& P, int h, int& q, int ticket) {
    const int it = ticket * NQUEUE + q;
    return it < P.N ? it : queue_pop(P, h, q);
}
__device__ __forceinline__ int first_queue(int H) { return ((int)blockIdx.x / H) % NQUEUE; }

// ---- item records ------------------------------------------------------------------------------
// Everything a wavefront needs to start on item (it, h), gathered by prepare_items_kernel into one
// 128-byte record so that the main kernels fetch it with ONE coalesced load, issued a whole item
// ahead (the chain order -> batch -> lattice would be three dependent round trips per item):
//   word 0 atom i, 1 first pair, 2 number of pairs, 3 R1 | R2 << 8 | R3 << 16, 4 a_ih,
//   5..13 lattice rows, 14..22 frame axes (frame search: 14..29 the query vector q_ih),
//   30 first neighbour atom (the pairs of an atom point at consecutive atoms), 31 crystal
constexpr int REC_WORDS = 32;
constexpr int SLOW_PREP_SLOTS = 256;           // slots of a list of slow records: every record of the block that makes it
constexpr uint32_t REC_BOX_LISTED = 0x80000000u;      // flag in the box word of a record listed by the launch that made it
constexpr uint32_t REC_BOX_LISTED_BWD = 0x40000000u;  // ... listed again for the backward pass (see core_gbuild_kernel)
enum { REC_ATOM = 0, REC_E0 = 1, REC_NPAIRS = 2, REC_BOX = 3, REC_A = 4, REC_LATTICE = 5, REC_FRAMES = 14,
       REC_QUERY = 14 };

struct Item {
    int i, e0, npairs;
    float a;
    Box bx;
    Lattice L;
};
__device__ __forceinline__ float rec_f(uint32_t rec, int word) {
    return __int_as_float(__builtin_amdgcn_readlane((int)rec, word));
}
__device__ __forceinline__ Item unpack_item(uint32_t rec) {
    Item t;
    t.i = __builtin_amdgcn_readlane((int)rec, REC_ATOM);
    t.e0 = __builtin_amdgcn_readlane((int)rec, REC_E0);
    t.npairs = __builtin_amdgcn_readlane((int)rec, REC_NPAIRS);
    const int box = __builtin_amdgcn_readlane((int)rec, REC_BOX);
    t.bx.R1 = box & 255; t.bx.R2 = (box >> 8) & 255; t.bx.R3 = (box >> 16) & 255;
    t.bx.s2 = 2 * t.bx.R2 + 1; t.bx.s3 = 2 * t.bx.R3 + 1;
    t.bx.T = (2 * t.bx.R1 + 1) * t.bx.s2 * t.bx.s3;
    t.bx.over = 0;
    t.a = rec_f(rec, REC_A);
#pragma unroll
    for (int d = 0; d < 9; d++) t.L.t[d] = rec_f(rec, REC_LATTICE + d);
    return t;
}
// the same for a wavefront that is not the first of its workgroup
// wid / H without a division (the heads are a launch argument, and a 32-bit division is some 25 vector instructions)
__device__ __forceinline__ int div_heads(const KernelArgs& P, int wid) {
    return P.h_magic ? (int)(__umulhi((uint32_t)wid, P.h_magic) >> P.h_shift) : wid;
}
__device__ __forceinline__ uint32_t load_record_lane(const KernelArgs& P, int it, int h, int lane) {
    return (it >= 0 && lane < REC_WORDS) ? P.items[((size_t)it * P.H + h) * REC_WORDS + lane] : 0u;
}
__device__ __forceinline__ uint32_t load_record(const KernelArgs& P, int it, int h) {
    return (it >= 0 && threadIdx.x < REC_WORDS) ? P.items[((size_t)it * P.H + h) * REC_WORDS + threadIdx.x] : 0u;
}

// One thread per (item, head): builds the records, clears the work queues of the launch and (backward)
// the weight-gradient outputs that the reduction after the main kernel adds into.
__device__ __forceinline__ void prepare_items_block(const KernelArgs& P, int with_query, int block) {
    const int idx = block * 256 + (int)threadIdx.x;
    if (idx < P.H * NQUEUE) {
        P.counters[idx * QSTRIDE] = 0;
        if (P.counters2) P.counters2[idx * QSTRIDE] = 0;
    }
    if (idx == 0 && with_query && P.seed_dev) {
        const unsigned long long s = *P.seed_dev;
        *P.seed_snap = s;
        if (P.seed_advance) *P.seed_dev = s + 1ull;
    }
    if (idx < P.gw_out_n) {
#pragma unroll
        for (int en = 0; en < 4; en++)
            if (P.gw_out[en]) P.gw_out[en][idx] = 0.0f;
    }
    const bool valid = idx < P.N * P.H;
    bool slow = false;
    uint32_t* rec = P.items + (size_t)(valid ? idx : 0) * REC_WORDS;
    uint32_t boxw = 0;
    if (valid) {
        const int it = idx / P.H, h = idx - it * P.H;
        const int i = P.order ? P.order[it] : it;
        const int b = (int)P.batch[i];
        const float a = P.a_ih[(size_t)i * P.H + h];
        float rvl1 = 0.f, rvl2 = 0.f, rvl3 = 0.f;
        if (P.rvlen) { rvl1 = P.rvlen[(size_t)b * 3 + 0]; rvl2 = P.rvlen[(size_t)b * 3 + 1]; rvl3 = P.rvlen[(size_t)b * 3 + 2]; }
        const Box bx = translation_box(a, rvl1, rvl2, rvl3, P.cutoff_radius, P.lattice_range, P.minimum_range);
        if (bx.over && P.status) atomicOr(P.status, 1);
        const int e0 = (int)P.e_start[i];
        rec[REC_ATOM] = (uint32_t)i;
        rec[REC_E0] = (uint32_t)e0;
        rec[REC_NPAIRS] = (uint32_t)((int)P.e_start[i + 1] - e0);
        boxw = (uint32_t)(bx.R1 | (bx.R2 << 8) | (bx.R3 << 16));
        slow = P.slow_count != nullptr && !(bx.R1 == P.slow_R && bx.R2 == P.slow_R && bx.R3 == P.slow_R);
        rec[REC_A] = __float_as_uint(a);
        for (int d = 0; d < 9; d++) rec[REC_LATTICE + d] = __float_as_uint(P.tvecs[(size_t)b * 9 + d]);
        int j0 = P.e_start[i + 1] > e0 ? (int)P.edges[(size_t)P.E + e0] : i;      // first neighbour atom
        if (P.contiguous_neighbours) {
            // a layout other than whole n x n blocks would make the kernels read other atoms than the pairs name, or
            // past the last atom: say so in the status word and keep every read inside the arrays
            const int np = (int)P.e_start[i + 1] - e0;
            const bool bad = j0 < 0 || j0 + np > P.N || (np > 0 && (int)P.edges[(size_t)P.E + e0 + np - 1] != j0 + np - 1);
            if (bad) {
                if (P.status) atomicOr(P.status, 2);
                j0 = max(0, min(j0, P.N - np));
            }
        }
        rec[30] = (uint32_t)j0;
        rec[31] = (uint32_t)b;                                                                  // crystal
        if (with_query) {
            for (int c = 0; c < DH; c++) rec[REC_QUERY + c] = __float_as_uint(P.q[((size_t)i * P.H + h) * DH + c]);
        } else if (P.frames) {
            for (int ax = 0; ax < 3; ax++)
                for (int d = 0; d < 3; d++)
                    rec[REC_FRAMES + ax * 3 + d] = __float_as_uint(P.frames[(((size_t)ax * P.N + i) * P.H + h) * 3 + d]);
        }
    }
    // The records whose box is not the usual one take several times as long as the others in the kernels that
    // follow, and most of them are atoms of small crystals at the END of the work order, where they alone make the
    // tail of a launch.  The block lists its own (rank by ballot, no atomics, nothing to clear); a launch that wants
    // them first starts with a few wavefronts that take the listed records by their rank over all lists, and skips a
    // listed record in its place.
    if (P.slow_count) {
        __shared__ int slow_in_wave[4];
        const int ln = threadIdx.x & (WAVE - 1), wv = threadIdx.x >> 6;
        const uint64_t m = ballot(slow);
        if (ln == 0) slow_in_wave[wv] = __popcll(m);
        __syncthreads();
        int rank = __popcll(m & ((1ull << ln) - 1ull)), total = 0;
        for (int w = 0; w < 4; w++) { rank += w < wv ? slow_in_wave[w] : 0; total += slow_in_wave[w]; }
        if (slow) {
            P.slow_list[block * SLOW_PREP_SLOTS + rank] = idx;
            boxw |= REC_BOX_LISTED;
        }
        if (threadIdx.x == 0) P.slow_count[block] = total;
    }
    if (valid) rec[REC_BOX] = boxw;
}
__global__ __launch_bounds__(256) void prepare_items_kernel(const KernelArgs P, int with_query) {
    prepare_items_block(P, with_query, (int)blockIdx.x);
}

// Counter-based uniform in [0,1) for the optional tie-breaking noise of the frame search.
__device__ __forceinline__ float hash_uniform(uint32_t a, uint32_t b, uint32_t c, uint32_t d) {
    uint32_t x = a * 0x9E3779B1u ^ (b + 0x7F4A7C15u) * 0x85EBCA77u;
    x ^= x >> 15; x *= 0xC2B2AE3Du; x ^= c * 0x27D4EB2Fu; x ^= x >> 13; x *= 0x165667B1u;
    x ^= d; x ^= x >> 16; x *= 0x9E3779B1u; x ^= x >> 15;
    return (float)(x >> 8) * (1.0f / 16777216.0f);
}

}  // namespace cfh
