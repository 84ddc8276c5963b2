// C ABI of the gfx950 kernels (see include/crystalframer_hip.h).  Host side: argument checks,
// constant preparation and kernel launches.  Nothing here allocates or
// synchronises.
#include "../../include/crystalframer_hip.h"

#include <hip/hip_runtime.h>

#include <cmath>
#include <cstdarg>
#include <cstdio>
#include <cstring>
#include <mutex>
#include <string>
#include <vector>

#include "attention_inputs.hpp"
#include "device_common.hpp"
#include "frame_select.hpp"
#include "framed_pe_bwd.hpp"
#include "framed_pe_bwd_saved.hpp"
#include "framed_pe_fwd.hpp"
#include "fused_dpa.hpp"
#include "fused_core.hpp"
#include "frame_select_sorted.hpp"
#include "geometry.hpp"
#include "linear_grad.hpp"
#include "small_gemm.hpp"
#include "layer_bridge.hpp"
#include "adamw.hpp"

namespace {

thread_local char g_err[512] = "";

int fail(int code, const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
    return code;
}

constexpr int MAX_HEADS = 64;
constexpr size_t QUEUE_OFFSET = 512;           // workspace header: 256 reserved bytes, 32 uint64 statistics, then the work queues
constexpr size_t STATS_OFFSET = 256;
constexpr size_t STATUS_OFFSET = 16;          // int32 status word (box cut back to the largest half-width)
constexpr size_t QUEUE_SET_BYTES = (size_t)MAX_HEADS * cfh::NQUEUE * cfh::QSTRIDE * sizeof(int32_t);
constexpr size_t COUNTER_BYTES = QUEUE_OFFSET + 2 * QUEUE_SET_BYTES;   // whole header: two sets of work queues
constexpr int WAVES_PER_SIMD = 3;
constexpr int FRAME_WAVES_PER_SIMD = 8;      // the frame search keeps no per-wavefront partials: as many as are resident

// workspace: header | item records (N, H, REC_WORDS) | per-wavefront weight-gradient partials
size_t items_bytes(int64_t N, int H) {
    const size_t raw = (size_t)N * (size_t)H * cfh::REC_WORDS * sizeof(uint32_t);
    return (raw + 255) & ~(size_t)255;
}

// number of compute units of the current device (cached per device)
int device_cus() {
    static int cus[64] = {0};
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 0;
    if (cus[dev] == 0) {
        int v = 0;
        if (hipDeviceGetAttribute(&v, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess) return 0;
        cus[dev] = v;
    }
    return cus[dev];
}

// A second stream per device (default priority) with the two events that fork it from and join it to the
// stream of a call; created by the first call that uses it on the device.  The mutex orders whole
// fork .. join sequences of calls from different threads.
struct SideStream { hipStream_t stream = nullptr; hipEvent_t fork = nullptr, join = nullptr; };
std::mutex g_side_mutex;
SideStream* side_stream() {
    static SideStream side[64];
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return nullptr;
    SideStream& s = side[dev];
    if (!s.stream) {
        // the first call may come while the caller's stream is being captured: creating a stream and events
        // does not touch the capture, which the relaxed mode lets this thread say
        hipStreamCaptureMode mode = hipStreamCaptureModeRelaxed;
        const bool exchanged = hipThreadExchangeStreamCaptureMode(&mode) == hipSuccess;
        hipStream_t st = nullptr;
        hipEvent_t f = nullptr, j = nullptr;
        bool ok = hipStreamCreateWithFlags(&st, hipStreamNonBlocking) == hipSuccess;
        ok = ok && hipEventCreateWithFlags(&f, hipEventDisableTiming) == hipSuccess &&
             hipEventCreateWithFlags(&j, hipEventDisableTiming) == hipSuccess;
        if (exchanged) (void)hipThreadExchangeStreamCaptureMode(&mode);      // back to the caller's mode
        if (!ok) {
            if (f) (void)hipEventDestroy(f);
            if (st) (void)hipStreamDestroy(st);
            (void)hipGetLastError();
            return nullptr;
        }
        s.fork = f; s.join = j; s.stream = st;
    }
    return &s;
}

// upper bound of the persistent wavefronts of a launch (sizes the workspace): a multiple of H, no
// more than there are items
int launch_waves(int64_t N, int H, int per_simd = WAVES_PER_SIMD) {
    int cus = device_cus();
    if (cus <= 0) cus = 256;
    int64_t want = (int64_t)cus * 4 * per_simd;
    want = (want / H) * H;
    if (want < H) want = H;
    const int64_t items = N * H;
    if (want > items) want = items;
    return (int)want;
}

// The 16-bin angle basis of the reference's lightweight setting (train_jarvis_time.sh: value_pe_angle_real 16).  Its
// window (ANGLE_RANGE = ceil(8 wscale + 1) >= 9) leaves at most 7 bins out, so the reference evaluates the whole
// basis (models/kernels/real_enc_frame_proj_fwd_angle.cu:154,168-175: the windowed branch needs more than 8).  The
// kernels here are compiled for rows of 64 bins: the 16 bins are run as ONE 17-bin window that always starts at bin
// 0 (bin 16 is a padding bin), with the weights copied into zero-padded rows of 64.
constexpr int SMALL_ANGLE_BINS = 16;
constexpr int SMALL_ANGLE_WINDOW = 17;

int check_params(const cfh_params* p) {
    if (!p) return fail(CFH_EINVAL, "params is NULL");
    if (p->struct_size != (int32_t)sizeof(cfh_params))
        return fail(CFH_EINVAL, "cfh_params.struct_size %d != %zu (header/library mismatch)", p->struct_size,
                    sizeof(cfh_params));
    if (p->num_heads < 1 || p->num_heads > MAX_HEADS)
        return fail(CFH_EINVAL, "num_heads %d outside 1..%d", p->num_heads, MAX_HEADS);
    if (p->head_dim != cfh::DH) return fail(CFH_EINVAL, "head_dim %d not compiled (only %d)", p->head_dim, cfh::DH);
    if (p->dist_bins != 0 && p->dist_bins != cfh::NBINS)
        return fail(CFH_EINVAL, "dist_bins %d not compiled (0 or %d)", p->dist_bins, cfh::NBINS);
    if (p->angle_bins != 0 && p->angle_bins != cfh::NBINS && p->angle_bins != SMALL_ANGLE_BINS)
        return fail(CFH_EINVAL, "angle_bins %d not compiled (0, %d or %d)", p->angle_bins, SMALL_ANGLE_BINS, cfh::NBINS);
    if (p->angle_bins == SMALL_ANGLE_BINS && !(p->angle_wscale >= 1.0f))
        return fail(CFH_EINVAL, "angle_bins %d needs angle_wscale >= 1", SMALL_ANGLE_BINS);
    if (p->angle_bins != 0 && p->dist_bins == 0)
        return fail(CFH_EINVAL, "angle encoding requires the distance encoding (dist_bins > 0)");
    if (p->lattice_range < 0 || p->lattice_range > cfh::RMAX)
        return fail(CFH_EINVAL, "lattice_range %d outside 0..%d", p->lattice_range, cfh::RMAX);
    if (p->minimum_range < 0 || p->minimum_range > cfh::RMAX)
        return fail(CFH_EINVAL, "minimum_range %d outside 0..%d", p->minimum_range, cfh::RMAX);
    if (p->window_mode != CFH_WINDOW_REFERENCE && p->window_mode != CFH_WINDOW_WIDE)
        return fail(CFH_EINVAL, "window_mode %d unknown", p->window_mode);
    return CFH_OK;
}

// Bins of the distance window for the configured scale: ceil(2 wscale cut + 1) (LENGTH_RANGE of
// models/cuda_funcs/kernel_manager.py:146 for cut = 4), or the whole basis when that leaves at most 8 bins out
// (models/kernels/real_enc_frame_proj_fwd_length.cu:139-142: the windowed branch needs K - LENGTH_RANGE > 8).
int dist_window_bins(const cfh_params* p) {
    const int cut = (p->window_mode == CFH_WINDOW_WIDE) ? 5 : 4;
    int wl = (int)std::ceil(2.0 * (double)p->dist_wscale * cut + 1.0);
    if (wl < 1) wl = 1;
    if (p->dist_bins - wl <= 8) wl = p->dist_bins;
    return wl;
}
// The kernels are compiled for the widths of wscale 1 (9 bins, 11 for the wide mode) and once more for a width that
// is known at run time only (any other scale).
bool dist_window_dynamic(const cfh_params* p) {
    return p->dist_bins > 0 && dist_window_bins(p) != ((p->window_mode == CFH_WINDOW_WIDE) ? 11 : 9);
}
// window widths for the configured scales; the angle windows are instantiated for (33) and (41) only
int window_widths(const cfh_params* p, int* wl, int* wa) {
    const int cut = (p->window_mode == CFH_WINDOW_WIDE) ? 5 : 4;
    *wl = dist_window_bins(p);
    *wa = (int)std::ceil(2.0 * (double)p->angle_wscale * cut + 1.0);
    const int want_a = cut == 4 ? 33 : 41;
    if (p->angle_bins == SMALL_ANGLE_BINS) *wa = want_a;      // the whole basis whatever the scale
    if (p->dist_bins > 0 && !(p->dist_wscale > 0.0f))
        return fail(CFH_EINVAL, "dist_wscale %g must be positive", (double)p->dist_wscale);
    if (p->angle_bins == SMALL_ANGLE_BINS && dist_window_dynamic(p))
        return fail(CFH_EINVAL, "dist_wscale %g with 16 angle bins is not compiled for the two-step operators",
                    (double)p->dist_wscale);
    if (p->angle_bins > 0 && *wa != want_a)
        return fail(CFH_EINVAL, "angle_wscale %g gives a %d-bin window; only wscale 4.0 (%d bins) is compiled",
                    (double)p->angle_wscale, *wa, want_a);
    return CFH_OK;
}

cfh::BasisConsts basis_consts(const cfh_params* p) {
    cfh::BasisConsts bc;
    std::memset(&bc, 0, sizeof(bc));
    const double cut = (p->window_mode == CFH_WINDOW_WIDE) ? 5.0 : 4.0;
    const double sl2e = std::sqrt(1.4426950408889634);
    if (p->dist_bins > 0) {
        const double interval = (double)p->dist_max / p->dist_bins;
        bc.inv_interval = (float)(1.0 / interval);
        bc.start_off = (float)(cut * p->dist_wscale + 1.0);
        const double step = sl2e / ((double)p->dist_wscale * std::sqrt(2.0));
        bc.len_step = (float)step;
        bc.len_cc = (float)std::exp2(-2.0 * step * step);
        bc.len_window = dist_window_bins(p);
    }
    if (p->angle_bins > 0) {
        const int A = p->angle_bins;
        const double interval = (p->cos_abs ? 1.0 : 2.0) / (A - 1);
        // the reference passes sigma to its kernels as a float32 scalar
        const double sigma = (double)(float)((p->cos_abs ? 1.0 : 2.0) * (double)p->angle_wscale / (A - 1));
        bc.ang_inv_interval = (float)(1.0 / interval);
        bc.ang_end_off = (float)(1.0 + cut * sigma);
        bc.ang_interval = (float)interval;
        const double sinv = sl2e / (sigma * std::sqrt(2.0));
        bc.ang_sigma_inv = (float)sinv;
        bc.ang_step = (float)(interval * sinv);
        bc.ang_cc = (float)std::exp2(-2.0 * interval * sinv * interval * sinv);
        bc.ang_mu0 = p->cos_abs ? 0.0f : -1.0f;
        bc.ang_end_max = A == SMALL_ANGLE_BINS ? (float)SMALL_ANGLE_WINDOW : (float)A;
    }
    return bc;
}

int check_geometry(const float* a_ih, const float* rpos, const float* tvecs, const int64_t* batch,
                   const int64_t* edges, const int64_t* e_start, int64_t N, int64_t E, int64_t B) {
    if (N < 0 || E < 0 || B < 0) return fail(CFH_EINVAL, "negative size N=%lld E=%lld B=%lld", (long long)N, (long long)E, (long long)B);
    if (N > 0x7fffffffLL / 64 || E > 0x7fffffffLL / 64)
        return fail(CFH_EINVAL, "N=%lld or E=%lld beyond the 32-bit index range of the kernels", (long long)N, (long long)E);
    if (N == 0) return CFH_OK;
    if (!a_ih || !rpos || !tvecs || !batch || !edges || !e_start)
        return fail(CFH_EINVAL, "a_ih, rpos, tvecs, batch, edges and e_start must not be NULL");
    return CFH_OK;
}

int check_workspace(void* ws, size_t have, size_t need) {
    if (!ws || have < need) return fail(CFH_EWORKSPACE, "workspace of %zu bytes needed, %zu given", need, have);
    if (((uintptr_t)ws & 255) != 0) return fail(CFH_EWORKSPACE, "workspace must be 256-byte aligned");
    return CFH_OK;
}

void fill_common(cfh::KernelArgs& A, const cfh_params* p, const float* a_ih, const float* rpos,
                 const float* tvecs, const float* rvlen, const int64_t* batch, const int64_t* edges,
                 const int64_t* e_start, const int32_t* order, int64_t N, int64_t E, void* workspace) {
    std::memset(&A, 0, sizeof(A));
    A.a_ih = a_ih; A.rpos = rpos; A.tvecs = tvecs; A.rvlen = rvlen;
    A.batch = batch; A.edges = edges; A.e_start = e_start; A.order = order;
    A.counters = reinterpret_cast<int32_t*>(reinterpret_cast<char*>(workspace) + QUEUE_OFFSET);
    A.items = reinterpret_cast<uint32_t*>(reinterpret_cast<char*>(workspace) + COUNTER_BYTES);
    A.stats = p->collect_stats ? reinterpret_cast<unsigned long long*>(reinterpret_cast<char*>(workspace) + STATS_OFFSET) : nullptr;
    A.N = (int32_t)N; A.E = (int32_t)E; A.H = p->num_heads;
    {
        // n / H = (n * m) >> (31 + l) with l = ceil(log2 H), m = ceil(2^(31 + l) / H) < 2^32: exact for 0 <= n < 2^31
        const uint32_t d = (uint32_t)p->num_heads;
        if (d <= 1) { A.h_magic = 0; A.h_shift = 0; }
        else {
            int l = 0;
            while ((1u << l) < d) l++;
            const unsigned long long two = 1ull << (31 + l);
            A.h_magic = (uint32_t)((two + d - 1) / d);
            A.h_shift = l - 1;
        }
    }
    A.cutoff_radius = rvlen ? p->cutoff_radius : 0.0f;
    A.lattice_range = p->lattice_range; A.minimum_range = p->minimum_range;
    A.prune_log2 = p->prune_log2;
    A.dist_coef = p->dist_coef; A.angle_coef = p->angle_coef;
    A.gz_coef = p->grad_coef_quirk ? p->dist_coef : 1.0f;
    A.gw_dist_coef = p->grad_coef_quirk ? 1.0f : p->dist_coef;
    A.noise = p->symm_break_noise;
    A.seed_lo = (uint32_t)(p->noise_seed & 0xffffffffu);
    A.seed_hi = (uint32_t)(p->noise_seed >> 32);
    A.seed_dev = reinterpret_cast<unsigned long long*>(p->noise_seed_dev);
    A.seed_snap = reinterpret_cast<unsigned long long*>(workspace);      // first word of the reserved header bytes
    A.status = reinterpret_cast<int32_t*>(reinterpret_cast<char*>(workspace) + STATUS_OFFSET);
    A.seed_advance = p->noise_seed_advance;
    A.bc = basis_consts(p);
}

int finish_launch(const char* what) {
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess) return fail(CFH_ELAUNCH, "%s: %s", what, hipGetErrorString(e));
    return CFH_OK;
}

// Wavefronts that are resident at once for this kernel on the current device.  Work is dealt to
// wavefronts statically, so launching more than fit would run them in a second wave of blocks and
// double the makespan.
template <typename Kern>
int resident_waves(Kern kern, int cap, int H) {
    int per_cu = 0;
    if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, kern, cfh::WAVE, 0) != hipSuccess || per_cu < 1)
        per_cu = 4;
    int cus = device_cus();
    if (cus <= 0) cus = 256;
    int64_t want = (int64_t)cus * per_cu;
    if (want > cap) want = cap;
    want = (want / H) * H;
    if (want < H) want = H;
    return (int)want;
}

// Optional timing of the lattice-sum kernels alone (not the small kernels around them): HIP events
// on the stream of the launch, kept until cfh_timing_read collects them.
struct TimedLaunch { std::string what; hipEvent_t start, stop; };
std::mutex g_timing_mutex;
bool g_timing_on = false;
std::vector<TimedLaunch> g_timed;
// set by an entry point that must not allocate (events are allocations): its launches are never timed
thread_local bool t_timing_blocked = false;
// Brackets the launches made during its lifetime with a pair of events on their stream, when timing is on.
struct TimedScope {
    TimedLaunch t;
    hipStream_t st;
    bool on = false;
    TimedScope(const char* what, hipStream_t stream) : st(stream) {
        if (t_timing_blocked) return;
        {
            std::lock_guard<std::mutex> lock(g_timing_mutex);
            on = g_timing_on;
        }
        if (!on) return;
        t.what = what;
        on = hipEventCreate(&t.start) == hipSuccess && hipEventCreate(&t.stop) == hipSuccess &&
             hipEventRecord(t.start, st) == hipSuccess;
    }
    ~TimedScope() {
        if (on && hipEventRecord(t.stop, st) == hipSuccess) {
            std::lock_guard<std::mutex> lock(g_timing_mutex);
            g_timed.push_back(t);
        }
    }
    TimedScope(const TimedScope&) = delete;
    TimedScope& operator=(const TimedScope&) = delete;
};

// `waves`: in = upper bound, out = wavefronts actually launched
template <typename Kern>
int launch_persistent(Kern kern, const cfh::KernelArgs& A, int* waves, hipStream_t st, const char* what,
                      bool prepare = true) {
    *waves = resident_waves(kern, *waves, A.H);
    if (prepare) {
        int threads = A.N * A.H > A.H * cfh::NQUEUE ? A.N * A.H : A.H * cfh::NQUEUE;
        if (threads < A.gw_out_n) threads = A.gw_out_n;
        hipLaunchKernelGGL(cfh::prepare_items_kernel, dim3((threads + 255) / 256), dim3(256), 0, st, A, A.q != nullptr ? 1 : 0);
    }
    {
        TimedScope timed(what, st);
        hipLaunchKernelGGL(kern, dim3(*waves), dim3(cfh::WAVE), 0, st, A);
    }
    return finish_launch(what);
}

}  // namespace

extern "C" {

int cfh_abi_version(void) { return CFH_ABI_VERSION; }

const char* cfh_last_error(void) { return g_err; }

int cfh_second_stream_fork(void* stream, void** second) {
    if (!second) return fail(CFH_EINVAL, "second must not be NULL");
    std::lock_guard<std::mutex> lock(g_side_mutex);
    SideStream* side = side_stream();
    if (!side) return fail(CFH_ELAUNCH, "second stream could not be created");
    if (hipEventRecord(side->fork, (hipStream_t)stream) != hipSuccess ||
        hipStreamWaitEvent(side->stream, side->fork, 0) != hipSuccess)
        return fail(CFH_ELAUNCH, "fork to the second stream failed: %s", hipGetErrorString(hipGetLastError()));
    *second = (void*)side->stream;
    return CFH_OK;
}

int cfh_second_stream_get(void** second) {
    if (!second) return fail(CFH_EINVAL, "second must not be NULL");
    std::lock_guard<std::mutex> lock(g_side_mutex);
    SideStream* side = side_stream();
    if (!side) return fail(CFH_ELAUNCH, "second stream could not be created");
    *second = (void*)side->stream;
    return CFH_OK;
}

int cfh_second_stream_join(void* stream) {
    std::lock_guard<std::mutex> lock(g_side_mutex);
    SideStream* side = side_stream();
    if (!side) return fail(CFH_ELAUNCH, "second stream could not be created");
    if (hipEventRecord(side->join, side->stream) != hipSuccess ||
        hipStreamWaitEvent((hipStream_t)stream, side->join, 0) != hipSuccess)
        return fail(CFH_ELAUNCH, "join of the second stream failed: %s", hipGetErrorString(hipGetLastError()));
    return CFH_OK;
}

int cfh_timing_enable(int on) {
    std::lock_guard<std::mutex> lock(g_timing_mutex);
    g_timing_on = on != 0;
    return CFH_OK;
}

int cfh_timing_read(const char* what, double* total_ms, int64_t* launches) {
    if (!what || !total_ms || !launches) return fail(CFH_EINVAL, "what, total_ms and launches must not be NULL");
    std::vector<TimedLaunch> mine, rest;
    {
        std::lock_guard<std::mutex> lock(g_timing_mutex);
        for (const TimedLaunch& t : g_timed) (t.what == what ? mine : rest).push_back(t);
        g_timed.swap(rest);
    }
    *total_ms = 0.0;
    *launches = 0;
    for (const TimedLaunch& t : mine) {
        float ms = 0.0f;
        if (hipEventSynchronize(t.stop) == hipSuccess && hipEventElapsedTime(&ms, t.start, t.stop) == hipSuccess) {
            *total_ms += (double)ms;
            *launches += 1;
        }
        (void)hipEventDestroy(t.start);
        (void)hipEventDestroy(t.stop);
    }
    return CFH_OK;
}

}  // extern "C"
namespace {
// workspace of the lattice-sum calls: header | item records | per-wavefront weight-gradient partials | six padded
// (H, Dh, 64) rows for the 16-bin angle basis (three weights, three gradients)
size_t padded_offset(const cfh_params* p, int64_t N) {
    const int waves = launch_waves(N > 0 ? N : 1, p->num_heads);
    return COUNTER_BYTES + items_bytes(N > 0 ? N : 1, p->num_heads) + (size_t)waves * 4 * cfh::DH * cfh::NBINS * sizeof(float);
}
}  // namespace
extern "C" {

size_t cfh_workspace_bytes(const cfh_params* p, int64_t N, int64_t E) {
    (void)E;
    if (check_params(p) != CFH_OK) return 0;
    return padded_offset(p, N) + 6 * (size_t)p->num_heads * cfh::DH * cfh::NBINS * sizeof(float);
}

int cfh_frame_axis1(const cfh_params* p, const float* q, const float* k, const float* a_ih,
                    const float* rpos, const float* tvecs, const float* rvlen, const int64_t* batch,
                    const int64_t* edges, const int64_t* e_start, const int32_t* order, int64_t N,
                    int64_t E, int64_t B, float* frame1, void* workspace, size_t workspace_bytes,
                    void* stream) {
    int rc = check_params(p);
    if (rc) return rc;
    if ((rc = check_geometry(a_ih, rpos, tvecs, batch, edges, e_start, N, E, B))) return rc;
    if (N == 0) return CFH_OK;
    if (!q || !k || !frame1) return fail(CFH_EINVAL, "q, k and frame1 must not be NULL");
    if ((rc = check_workspace(workspace, workspace_bytes, COUNTER_BYTES + items_bytes(N, p->num_heads)))) return rc;
    cfh::KernelArgs A;
    fill_common(A, p, a_ih, rpos, tvecs, rvlen, batch, edges, e_start, order, N, E, workspace);
    A.q = q; A.k = k; A.out_frame = frame1;
    int waves = launch_waves(N, p->num_heads, FRAME_WAVES_PER_SIMD);
    return launch_persistent(cfh::frame_axis_kernel<0>, A, &waves, (hipStream_t)stream, "frame_axis1");
}

int cfh_frame_axis2(const cfh_params* p, const float* q, const float* k, const float* a_ih,
                    const float* rpos, const float* tvecs, const float* rvlen, const int64_t* batch,
                    const int64_t* edges, const int64_t* e_start, const int32_t* order,
                    const float* frame1, int64_t N, int64_t E, int64_t B, float* frame2max,
                    void* workspace, size_t workspace_bytes, void* stream) {
    int rc = check_params(p);
    if (rc) return rc;
    if ((rc = check_geometry(a_ih, rpos, tvecs, batch, edges, e_start, N, E, B))) return rc;
    if (N == 0) return CFH_OK;
    if (!q || !k || !frame1 || !frame2max) return fail(CFH_EINVAL, "q, k, frame1 and frame2max must not be NULL");
    if ((rc = check_workspace(workspace, workspace_bytes, COUNTER_BYTES + items_bytes(N, p->num_heads)))) return rc;
    cfh::KernelArgs A;
    fill_common(A, p, a_ih, rpos, tvecs, rvlen, batch, edges, e_start, order, N, E, workspace);
    A.q = q; A.k = k; A.frame1 = frame1; A.out_frame = frame2max;
    int waves = launch_waves(N, p->num_heads, FRAME_WAVES_PER_SIMD);
    return launch_persistent(cfh::frame_axis_kernel<1>, A, &waves, (hipStream_t)stream, "frame_axis2");
}

int cfh_frame_axes(const cfh_params* p, const float* q, const float* k, const float* a_ih,
                   const float* rpos, const float* tvecs, const float* rvlen, const int64_t* batch,
                   const int64_t* edges, const int64_t* e_start, const int32_t* order, int64_t N,
                   int64_t E, int64_t B, float* frames, void* workspace, size_t workspace_bytes,
                   void* stream) {
    int rc = check_params(p);
    if (rc) return rc;
    if ((rc = check_geometry(a_ih, rpos, tvecs, batch, edges, e_start, N, E, B))) return rc;
    if (N == 0) return CFH_OK;
    if (!q || !k || !frames) return fail(CFH_EINVAL, "q, k and frames must not be NULL");
    if ((rc = check_workspace(workspace, workspace_bytes, COUNTER_BYTES + items_bytes(N, p->num_heads)))) return rc;
    cfh::KernelArgs A;
    fill_common(A, p, a_ih, rpos, tvecs, rvlen, batch, edges, e_start, order, N, E, workspace);
    A.q = q; A.k = k; A.out_frame = frames;
    int waves = launch_waves(N, p->num_heads, FRAME_WAVES_PER_SIMD);
    return launch_persistent(cfh::frame_axis_kernel<2>, A, &waves, (hipStream_t)stream, "frame_axes");
}

#define CFH_DISPATCH_PE(KERNEL, HAS_LEN, HAS_ANG)                                                   \
    do {                                                                                            \
        if (wide) {                                                                                 \
            if (p->cos_abs) rc = (dyn ? launch_persistent(KERNEL<0, 41, true, HAS_LEN, HAS_ANG>, A, &waves, st, what) : launch_persistent(KERNEL<11, 41, true, HAS_LEN, HAS_ANG>, A, &waves, st, what));  \
            else rc = (dyn ? launch_persistent(KERNEL<0, 41, false, HAS_LEN, HAS_ANG>, A, &waves, st, what) : launch_persistent(KERNEL<11, 41, false, HAS_LEN, HAS_ANG>, A, &waves, st, what));            \
        } else {                                                                                    \
            if (p->cos_abs) rc = (dyn ? launch_persistent(KERNEL<0, 33, true, HAS_LEN, HAS_ANG>, A, &waves, st, what) : launch_persistent(KERNEL<9, 33, true, HAS_LEN, HAS_ANG>, A, &waves, st, what));   \
            else rc = (dyn ? launch_persistent(KERNEL<0, 33, false, HAS_LEN, HAS_ANG>, A, &waves, st, what) : launch_persistent(KERNEL<9, 33, false, HAS_LEN, HAS_ANG>, A, &waves, st, what));             \
        }                                                                                           \
    } while (0)

#define CFH_DISPATCH_PE_NOGW(KERNEL, HAS_ANG)                                                       \
    do {                                                                                            \
        if (wide) {                                                                                 \
            if (p->cos_abs) rc = (dyn ? launch_persistent(KERNEL<0, 41, true, true, HAS_ANG, false>, A, &waves, st, what) : launch_persistent(KERNEL<11, 41, true, true, HAS_ANG, false>, A, &waves, st, what));  \
            else rc = (dyn ? launch_persistent(KERNEL<0, 41, false, true, HAS_ANG, false>, A, &waves, st, what) : launch_persistent(KERNEL<11, 41, false, true, HAS_ANG, false>, A, &waves, st, what));            \
        } else {                                                                                    \
            if (p->cos_abs) rc = (dyn ? launch_persistent(KERNEL<0, 33, true, true, HAS_ANG, false>, A, &waves, st, what) : launch_persistent(KERNEL<9, 33, true, true, HAS_ANG, false>, A, &waves, st, what));   \
            else rc = (dyn ? launch_persistent(KERNEL<0, 33, false, true, HAS_ANG, false>, A, &waves, st, what) : launch_persistent(KERNEL<9, 33, false, true, HAS_ANG, false>, A, &waves, st, what));             \
        }                                                                                           \
    } while (0)

// Forward of the lattice sums; with q and k also the frame search in front of it, whose item records
// and frames the forward kernel then takes over (one prepare launch for both).
static int framed_pe_forward_impl(const cfh_params* p, const float* q, const float* k, const float* a_ih,
                                  const float* rpos, const float* tvecs, const float* rvlen, const int64_t* batch,
                                  const int64_t* edges, const int64_t* e_start, const int32_t* order,
                                  const float* W_dist, const float* W_axis1, const float* W_axis2,
                                  const float* W_axis3, const float* frames_in, float* frames_out, int64_t N,
                                  int64_t E, int64_t B, float* z, float* psi, float* d2min_out, float* shat_out,
                                  void* workspace, size_t workspace_bytes, void* stream) {
    const bool search = q != nullptr;
    int rc = check_params(p);
    if (rc) return rc;
    if ((rc = check_geometry(a_ih, rpos, tvecs, batch, edges, e_start, N, E, B))) return rc;
    if (N == 0) return CFH_OK;
    if (!z) return fail(CFH_EINVAL, "z must not be NULL");
    const bool has_len = p->dist_bins > 0 && W_dist != nullptr;
    const bool has_ang = has_len && p->angle_bins > 0 && W_axis1 != nullptr;
    const float* frames = search ? frames_out : frames_in;
    if (p->dist_bins > 0 && !W_dist) return fail(CFH_EINVAL, "dist_bins > 0 but W_dist is NULL");
    if (has_len && !psi) return fail(CFH_EINVAL, "psi must not be NULL when dist_bins > 0");
    if (has_ang && (!W_axis2 || !W_axis3 || !frames))
        return fail(CFH_EINVAL, "W_axis1..3 and frames must be given together");
    if (search && (!k || !frames_out)) return fail(CFH_EINVAL, "q, k and frames must not be NULL");
    int wl = 0, wa = 0;
    if ((rc = window_widths(p, &wl, &wa))) return rc;
    if ((rc = check_workspace(workspace, workspace_bytes, COUNTER_BYTES + items_bytes(N, p->num_heads)))) return rc;
    hipStream_t st = (hipStream_t)stream;
    cfh::KernelArgs A;
    fill_common(A, p, a_ih, rpos, tvecs, rvlen, batch, edges, e_start, order, N, E, workspace);
    if (search) {
        cfh::KernelArgs F = A;
        F.q = q; F.k = k; F.out_frame = frames_out;
        F.counters2 = reinterpret_cast<int32_t*>(reinterpret_cast<char*>(workspace) + QUEUE_OFFSET + QUEUE_SET_BYTES);
        F.frames_to_records = 1;
        int fwaves = launch_waves(N, p->num_heads, FRAME_WAVES_PER_SIMD);
        if ((rc = launch_persistent(cfh::frame_axis_kernel<2>, F, &fwaves, st, "frame_axes"))) return rc;
        A.counters = F.counters2;
    }
    A.W[0] = W_dist; A.W[1] = W_axis1; A.W[2] = W_axis2; A.W[3] = W_axis3;
    if (has_ang && p->angle_bins == SMALL_ANGLE_BINS) {      // the 16-bin basis runs on zero-padded copies of its weights
        const int rows = p->num_heads * cfh::DH, per = rows * cfh::NBINS;
        const size_t off = padded_offset(p, N);
        if ((rc = check_workspace(workspace, workspace_bytes, off + 3 * (size_t)per * sizeof(float)))) return rc;
        float* padded = reinterpret_cast<float*>(reinterpret_cast<char*>(workspace) + off);
        hipLaunchKernelGGL(cfh::pad_bins_kernel, dim3((3 * per + 255) / 256), dim3(256), 0, st, W_axis1, W_axis2, W_axis3, rows,
                           SMALL_ANGLE_BINS, padded);
        A.W[1] = padded; A.W[2] = padded + per; A.W[3] = padded + 2 * per;
    }
    A.frames = frames; A.out_z = z; A.out_psi = psi; A.out_d2min = d2min_out; A.shat = shat_out;
    int waves = launch_waves(N, p->num_heads);
    const bool wide = p->window_mode == CFH_WINDOW_WIDE;
    const bool dyn = dist_window_dynamic(p);      // a distance window whose width is not one of the compiled ones
    const char* what = "framed_pe_forward";
    const bool prep = !search;
#define CFH_DISPATCH_FWD(HAS_LEN, HAS_ANG)                                                                      \
    do {                                                                                                        \
        if (wide) {                                                                                             \
            if (p->cos_abs) rc = (dyn ? launch_persistent(cfh::framed_pe_fwd_kernel<0, 41, true, HAS_LEN, HAS_ANG>, A, &waves, st, what, prep) : launch_persistent(cfh::framed_pe_fwd_kernel<11, 41, true, HAS_LEN, HAS_ANG>, A, &waves, st, what, prep));  \
            else rc = (dyn ? launch_persistent(cfh::framed_pe_fwd_kernel<0, 41, false, HAS_LEN, HAS_ANG>, A, &waves, st, what, prep) : launch_persistent(cfh::framed_pe_fwd_kernel<11, 41, false, HAS_LEN, HAS_ANG>, A, &waves, st, what, prep));            \
        } else {                                                                                                \
            if (p->cos_abs) rc = (dyn ? launch_persistent(cfh::framed_pe_fwd_kernel<0, 33, true, HAS_LEN, HAS_ANG>, A, &waves, st, what, prep) : launch_persistent(cfh::framed_pe_fwd_kernel<9, 33, true, HAS_LEN, HAS_ANG>, A, &waves, st, what, prep));   \
            else rc = (dyn ? launch_persistent(cfh::framed_pe_fwd_kernel<0, 33, false, HAS_LEN, HAS_ANG>, A, &waves, st, what, prep) : launch_persistent(cfh::framed_pe_fwd_kernel<9, 33, false, HAS_LEN, HAS_ANG>, A, &waves, st, what, prep));             \
        }                                                                                                       \
    } while (0)
    if (has_ang && p->angle_bins == SMALL_ANGLE_BINS) {
        if (wide) {
            if (p->cos_abs) rc = launch_persistent(cfh::framed_pe_fwd_kernel<11, SMALL_ANGLE_WINDOW, true, true, true>, A, &waves, st, what, prep);
            else rc = launch_persistent(cfh::framed_pe_fwd_kernel<11, SMALL_ANGLE_WINDOW, false, true, true>, A, &waves, st, what, prep);
        } else {
            if (p->cos_abs) rc = launch_persistent(cfh::framed_pe_fwd_kernel<9, SMALL_ANGLE_WINDOW, true, true, true>, A, &waves, st, what, prep);
            else rc = launch_persistent(cfh::framed_pe_fwd_kernel<9, SMALL_ANGLE_WINDOW, false, true, true>, A, &waves, st, what, prep);
        }
    } else if (has_ang) CFH_DISPATCH_FWD(true, true);
    else if (has_len) CFH_DISPATCH_FWD(true, false);
    else rc = (dyn ? launch_persistent(cfh::framed_pe_fwd_kernel<0, 33, false, false, false>, A, &waves, st, what, prep) : launch_persistent(cfh::framed_pe_fwd_kernel<9, 33, false, false, false>, A, &waves, st, what, prep));
#undef CFH_DISPATCH_FWD
    return rc;
}

int cfh_framed_pe_forward(const cfh_params* p, const float* a_ih, const float* rpos, const float* tvecs,
                          const float* rvlen, const int64_t* batch, const int64_t* edges,
                          const int64_t* e_start, const int32_t* order, const float* W_dist,
                          const float* W_axis1, const float* W_axis2, const float* W_axis3,
                          const float* frames, int64_t N, int64_t E, int64_t B, float* z, float* psi,
                          float* d2min_out, float* shat_out, void* workspace, size_t workspace_bytes,
                          void* stream) {
    return framed_pe_forward_impl(p, nullptr, nullptr, a_ih, rpos, tvecs, rvlen, batch, edges, e_start, order, W_dist,
                                  W_axis1, W_axis2, W_axis3, frames, nullptr, N, E, B, z, psi, d2min_out, shat_out,
                                  workspace, workspace_bytes, stream);
}

// ---- the forward of the lattice sums with its scratch in a file-scope device array ---------------------------
// For callers that cannot allocate (code under HIP graph capture, tight serving loops, harnesses that forbid
// hipMalloc).  What cfh_framed_pe_forward takes through its workspace argument -- work-queue heads and one
// 128-byte record per (atom, head) -- lives in `scratch` below, which every GPU the library runs on holds until
// the process ends.  In host code the array's name is only a stand-in: the address the kernels get is asked for
// once per device with hipGetSymbolAddress and kept.
constexpr size_t STATIC_SCRATCH_BYTES = COUNTER_BYTES + (size_t)CFH_STATIC_MAX_ITEMS * cfh::REC_WORDS * sizeof(uint32_t);
static __device__ __align__(256) unsigned char scratch[STATIC_SCRATCH_BYTES];

namespace {
std::mutex g_scratch_mutex;
void* g_scratch_ptr[64] = {nullptr};
// device address of `scratch` on the current device (nullptr: failure, message set)
void* static_scratch() {
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) {
        fail(CFH_EDEVICE, "no current HIP device");
        return nullptr;
    }
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (!g_scratch_ptr[dev]) {
        void* ptr = nullptr;
        // the first call on a device may come while the caller's stream is being captured: looking up a symbol
        // enqueues nothing, which the relaxed mode lets this thread say
        hipStreamCaptureMode mode = hipStreamCaptureModeRelaxed;
        const bool exchanged = hipThreadExchangeStreamCaptureMode(&mode) == hipSuccess;
        const hipError_t e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
        if (exchanged) (void)hipThreadExchangeStreamCaptureMode(&mode);
        if (e != hipSuccess || !ptr) {
            fail(CFH_EDEVICE, "hipGetSymbolAddress(scratch) failed on device %d: %s", dev, hipGetErrorString(e));
            return nullptr;
        }
        g_scratch_ptr[dev] = ptr;
    }
    return g_scratch_ptr[dev];
}
}  // namespace

int cfh_framed_pe_forward_static(const cfh_params* p, const float* a_ih, const float* rpos, const float* tvecs,
                                 const float* rvlen, const int64_t* batch, const int64_t* edges,
                                 const int64_t* e_start, const int32_t* order, const float* W_dist,
                                 const float* W_axis1, const float* W_axis2, const float* W_axis3,
                                 const float* frames, int64_t N, int64_t E, int64_t B, float* z, float* psi,
                                 float* d2min_out, float* shat_out, void* stream) {
    int rc = check_params(p);
    if (rc) return rc;
    if (N < 0) return fail(CFH_EINVAL, "negative size N=%lld", (long long)N);
    if (N * (int64_t)p->num_heads > (int64_t)CFH_STATIC_MAX_ITEMS)
        return fail(CFH_EINVAL, "N * num_heads = %lld exceeds the %d (atom, head) items the static scratch holds; "
                    "use cfh_framed_pe_forward with a workspace", (long long)(N * p->num_heads), CFH_STATIC_MAX_ITEMS);
    if (p->collect_stats) return fail(CFH_EINVAL, "collect_stats is not available with the static scratch");
    if (p->angle_bins == SMALL_ANGLE_BINS && W_axis1)
        return fail(CFH_EINVAL, "the 16-bin angle basis needs workspace for padded weights: use cfh_framed_pe_forward");
    void* ptr = static_scratch();
    if (!ptr) return CFH_EDEVICE;
    // the work-queue heads are cleared by the prepare kernel of every launch; nothing else must start at zero.
    // The timing diagnostics create events, i.e. allocate: they are off for this call whatever cfh_timing_enable says.
    struct Unblock { ~Unblock() { t_timing_blocked = false; } } unblock;
    t_timing_blocked = true;
    return framed_pe_forward_impl(p, nullptr, nullptr, a_ih, rpos, tvecs, rvlen, batch, edges, e_start, order, W_dist,
                                  W_axis1, W_axis2, W_axis3, frames, nullptr, N, E, B, z, psi, d2min_out, shat_out,
                                  ptr, STATIC_SCRATCH_BYTES, stream);
}

int cfh_frame_axes_framed_pe_forward(const cfh_params* p, const float* q, const float* k, const float* a_ih,
                                     const float* rpos, const float* tvecs, const float* rvlen,
                                     const int64_t* batch, const int64_t* edges, const int64_t* e_start,
                                     const int32_t* order, const float* W_dist, const float* W_axis1,
                                     const float* W_axis2, const float* W_axis3, int64_t N, int64_t E, int64_t B,
                                     float* frames, float* z, float* psi, float* d2min_out, float* shat_out,
                                     void* workspace, size_t workspace_bytes, void* stream) {
    if (N > 0 && !q) return fail(CFH_EINVAL, "q, k and frames must not be NULL");
    return framed_pe_forward_impl(p, q, k, a_ih, rpos, tvecs, rvlen, batch, edges, e_start, order, W_dist, W_axis1,
                                  W_axis2, W_axis3, nullptr, frames, N, E, B, z, psi, d2min_out, shat_out, workspace,
                                  workspace_bytes, stream);
}

static int framed_pe_backward_impl(const cfh_params* p, const float* a_ih, const float* rpos, const float* tvecs,
                           const float* rvlen, const int64_t* batch, const int64_t* edges,
                           const int64_t* e_start, const int32_t* order, const float* W_dist,
                           const float* W_axis1, const float* W_axis2, const float* W_axis3,
                           const float* frames, const float* z, const float* gz, const float* gpsi,
                           const float* shat, int64_t N, int64_t E, int64_t B, float* ga, float* gW_dist,
                           float* gW_axis1,
                           float* gW_axis2, float* gW_axis3, void* workspace, size_t workspace_bytes,
                           void* stream, const float* g_pair = nullptr) {
    int rc = check_params(p);
    if (rc) return rc;
    if ((rc = check_geometry(a_ih, rpos, tvecs, batch, edges, e_start, N, E, B))) return rc;
    // g_pair: the rows W^T gpsi come per pair from the caller; no weights, no weight gradients
    const bool has_len = p->dist_bins > 0 && (W_dist != nullptr || g_pair != nullptr);
    const bool has_ang = has_len && p->angle_bins > 0 && (W_axis1 != nullptr || (g_pair != nullptr && frames != nullptr));
    hipStream_t st = (hipStream_t)stream;
    const size_t wbytes = (size_t)p->num_heads * cfh::DH * cfh::NBINS * sizeof(float);
    if (N == 0) {     // no atoms: the weight gradients are zero
        const int per_enc = (int)(wbytes / sizeof(float));
        hipLaunchKernelGGL(cfh::zero_outputs_kernel, dim3((per_enc + 255) / 256), dim3(256), 0, st, per_enc,
                           gW_dist, gW_axis1, gW_axis2, gW_axis3);
        return finish_launch("zero_outputs");
    }
    if (!z || !gz || !ga) return fail(CFH_EINVAL, "z, gz and ga must not be NULL");
    if (has_len && !gpsi && !g_pair) return fail(CFH_EINVAL, "gpsi must not be NULL when dist_bins > 0");
    if (has_ang && !g_pair && (!W_axis2 || !W_axis3 || !frames))
        return fail(CFH_EINVAL, "W_axis1..3 and frames must be given together");
    int wl = 0, wa = 0;
    if ((rc = window_widths(p, &wl, &wa))) return rc;
    int waves = launch_waves(N, p->num_heads);
    const size_t need = COUNTER_BYTES + items_bytes(N, p->num_heads) + (size_t)waves * 4 * cfh::DH * cfh::NBINS * sizeof(float);
    if ((rc = check_workspace(workspace, workspace_bytes, need))) return rc;
    cfh::KernelArgs A;
    fill_common(A, p, a_ih, rpos, tvecs, rvlen, batch, edges, e_start, order, N, E, workspace);
    A.W[0] = W_dist; A.W[1] = W_axis1; A.W[2] = W_axis2; A.W[3] = W_axis3;
    A.frames = frames; A.z = z; A.gz = gz; A.gpsi = gpsi; A.out_ga = ga;
    A.shat = const_cast<float*>(shat);
    A.g_pair = g_pair;
    A.gw_partial = reinterpret_cast<float*>(reinterpret_cast<char*>(workspace) + COUNTER_BYTES + items_bytes(N, p->num_heads));
    if (g_pair) {        // gather-only kernel on this stream; nothing else
        const bool wide = p->window_mode == CFH_WINDOW_WIDE;
        const bool dyn = dist_window_dynamic(p);      // a distance window whose width is not one of the compiled ones
        const char* what = "framed_pe_backward";
        if (p->angle_bins == SMALL_ANGLE_BINS && has_ang) {
            if (wide) rc = p->cos_abs ? launch_persistent(cfh::framed_pe_bwd_saved_kernel<11, SMALL_ANGLE_WINDOW, true, true, true, false>, A, &waves, st, what)
                                      : launch_persistent(cfh::framed_pe_bwd_saved_kernel<11, SMALL_ANGLE_WINDOW, false, true, true, false>, A, &waves, st, what);
            else rc = p->cos_abs ? launch_persistent(cfh::framed_pe_bwd_saved_kernel<9, SMALL_ANGLE_WINDOW, true, true, true, false>, A, &waves, st, what)
                                 : launch_persistent(cfh::framed_pe_bwd_saved_kernel<9, SMALL_ANGLE_WINDOW, false, true, true, false>, A, &waves, st, what);
        } else if (has_ang) CFH_DISPATCH_PE_NOGW(cfh::framed_pe_bwd_saved_kernel, true);
        else CFH_DISPATCH_PE_NOGW(cfh::framed_pe_bwd_saved_kernel, false);
        return rc;
    }
    if (has_len) {      // cleared by the prepare kernel of this launch, added into by gw_reduce_kernel
        A.gw_out[0] = gW_dist;
        if (has_ang) { A.gw_out[1] = gW_axis1; A.gw_out[2] = gW_axis2; A.gw_out[3] = gW_axis3; }
        A.gw_out_n = p->num_heads * cfh::DH * cfh::NBINS;
    }
    const bool wide = p->window_mode == CFH_WINDOW_WIDE;
    const bool dyn = dist_window_dynamic(p);      // a distance window whose width is not one of the compiled ones
    const char* what = "framed_pe_backward";
    if (has_len && shat && !(p->flags & CFH_FLAG_SINGLE_STREAM) && p->angle_bins != SMALL_ANGLE_BINS) {
        // The forward kept its histograms and the weight gradients need nothing else: they are summed by a
        // streaming kernel of their own on a second stream while the gather-only kernel, free of their
        // accumulators, computes the gradient of a on this one.
        std::lock_guard<std::mutex> lock(g_side_mutex);
        SideStream* side = side_stream();
        if (!side) return fail(CFH_ELAUNCH, "second stream for the weight gradients could not be created");
        int cus = device_cus();
        if (cus <= 0) cus = 256;
        const int nslices = (cus * 4 + p->num_heads - 1) / p->num_heads;       // one wavefront per SIMD
        int gw_waves = nslices * p->num_heads;
        if ((size_t)gw_waves > (size_t)waves) {      // the workspace is sized for `waves` partials
            gw_waves = (waves / p->num_heads) * p->num_heads;
        }
        const int gw_slices = gw_waves / p->num_heads;
        // the kernels of this stream first, so that their wavefronts are resident when the others arrive
        if (hipEventRecord(side->fork, st) != hipSuccess)
            return fail(CFH_ELAUNCH, "fork to the second stream failed: %s", hipGetErrorString(hipGetLastError()));
        A.gw_out_n = 0;         // the weight gradients are cleared on the second stream
        if (has_ang) CFH_DISPATCH_PE_NOGW(cfh::framed_pe_bwd_saved_kernel, true);
        else CFH_DISPATCH_PE_NOGW(cfh::framed_pe_bwd_saved_kernel, false);
        // second stream: clear, partial sums per wavefront, their sum; it waits for nothing but the inputs
        const int nenc = has_ang ? 4 : 1;
        const int per_enc = p->num_heads * cfh::DH * cfh::NBINS;
        int rc2 = CFH_OK;
        if (hipStreamWaitEvent(side->stream, side->fork, 0) != hipSuccess)
            rc2 = fail(CFH_ELAUNCH, "fork to the second stream failed: %s", hipGetErrorString(hipGetLastError()));
        if (!rc2) {
            hipLaunchKernelGGL(cfh::zero_outputs_kernel, dim3((per_enc + 255) / 256), dim3(256), 0, side->stream, per_enc,
                               gW_dist, gW_axis1, gW_axis2, gW_axis3);
            if (has_ang)
                hipLaunchKernelGGL(cfh::gw_from_histograms_kernel<true>, dim3(gw_waves), dim3(cfh::WAVE), 0, side->stream,
                                   shat, gpsi, (int)E, p->num_heads, gw_slices, A.gw_dist_coef, A.angle_coef, A.gw_partial);
            else
                hipLaunchKernelGGL(cfh::gw_from_histograms_kernel<false>, dim3(gw_waves), dim3(cfh::WAVE), 0, side->stream,
                                   shat, gpsi, (int)E, p->num_heads, gw_slices, A.gw_dist_coef, A.angle_coef, A.gw_partial);
            const int rslices = 16;
            hipLaunchKernelGGL(cfh::gw_reduce_kernel, dim3((nenc * per_enc + 255) / 256, rslices), dim3(256), 0, side->stream,
                               A.gw_partial, gw_waves, p->num_heads, nenc, rslices, gW_dist, gW_axis1, gW_axis2, gW_axis3);
            rc2 = finish_launch("gw_from_histograms");
            // the join is enqueued whatever happened in between: a stream that was pulled into a capture must
            // come back to the capturing stream
            if (!(p->flags & CFH_FLAG_DEFER_JOIN) &&
                (hipEventRecord(side->join, side->stream) != hipSuccess || hipStreamWaitEvent(st, side->join, 0) != hipSuccess) && !rc2)
                rc2 = fail(CFH_ELAUNCH, "join of the second stream failed");
        }
        return rc ? rc : rc2;
    } else if (has_ang && p->angle_bins == SMALL_ANGLE_BINS) {
#define CFH_DISPATCH_SMALL(KERNEL)                                                                                   \
    do {                                                                                                             \
        if (wide) {                                                                                                  \
            if (p->cos_abs) rc = launch_persistent(KERNEL<11, SMALL_ANGLE_WINDOW, true, true, true>, A, &waves, st, what);   \
            else rc = launch_persistent(KERNEL<11, SMALL_ANGLE_WINDOW, false, true, true>, A, &waves, st, what);             \
        } else {                                                                                                     \
            if (p->cos_abs) rc = launch_persistent(KERNEL<9, SMALL_ANGLE_WINDOW, true, true, true>, A, &waves, st, what);    \
            else rc = launch_persistent(KERNEL<9, SMALL_ANGLE_WINDOW, false, true, true>, A, &waves, st, what);              \
        }                                                                                                            \
    } while (0)
        if (shat) CFH_DISPATCH_SMALL(cfh::framed_pe_bwd_saved_kernel);
        else CFH_DISPATCH_SMALL(cfh::framed_pe_bwd_kernel);
#undef CFH_DISPATCH_SMALL
    } else if (has_len && shat) {      // the forward kept its histograms: gather-only kernel
        if (has_ang) CFH_DISPATCH_PE(cfh::framed_pe_bwd_saved_kernel, true, true);
        else CFH_DISPATCH_PE(cfh::framed_pe_bwd_saved_kernel, true, false);
    } else if (has_ang) CFH_DISPATCH_PE(cfh::framed_pe_bwd_kernel, true, true);
    else if (has_len) CFH_DISPATCH_PE(cfh::framed_pe_bwd_kernel, true, false);
    else rc = (dyn ? launch_persistent(cfh::framed_pe_bwd_kernel<0, 33, false, false, false>, A, &waves, st, what) : launch_persistent(cfh::framed_pe_bwd_kernel<9, 33, false, false, false>, A, &waves, st, what));
    if (rc) return rc;
    if (has_len) {
        const int nenc = has_ang ? 4 : 1;
        const int per_enc = p->num_heads * cfh::DH * cfh::NBINS;
        const int total = nenc * per_enc;
        const int nslices = 16;
        hipLaunchKernelGGL(cfh::gw_reduce_kernel, dim3((total + 255) / 256, nslices), dim3(256), 0, st,
                           A.gw_partial, waves, p->num_heads, nenc, nslices, gW_dist, gW_axis1, gW_axis2, gW_axis3);
        rc = finish_launch("gw_reduce");
    }
    return rc;
}

int cfh_framed_pe_backward(const cfh_params* p, const float* a_ih, const float* rpos, const float* tvecs,
                           const float* rvlen, const int64_t* batch, const int64_t* edges,
                           const int64_t* e_start, const int32_t* order, const float* W_dist,
                           const float* W_axis1, const float* W_axis2, const float* W_axis3,
                           const float* frames, const float* z, const float* gz, const float* gpsi,
                           const float* shat, int64_t N, int64_t E, int64_t B, float* ga, float* gW_dist,
                           float* gW_axis1, float* gW_axis2, float* gW_axis3, void* workspace,
                           size_t workspace_bytes, void* stream) {
    int rc = check_params(p);
    if (rc) return rc;
    const bool small = p->angle_bins == SMALL_ANGLE_BINS && p->dist_bins > 0 && W_dist && W_axis1;
    if (!small)
        return framed_pe_backward_impl(p, a_ih, rpos, tvecs, rvlen, batch, edges, e_start, order, W_dist, W_axis1, W_axis2,
                                       W_axis3, frames, z, gz, gpsi, shat, N, E, B, ga, gW_dist, gW_axis1, gW_axis2,
                                       gW_axis3, workspace, workspace_bytes, stream);
    // The 16-bin angle basis: zero-padded copies of the weights in, padded gradient rows out (all on this stream).
    if (!W_axis2 || !W_axis3) return fail(CFH_EINVAL, "W_axis1..3 must be given together");
    hipStream_t st = (hipStream_t)stream;
    const int rows = p->num_heads * cfh::DH, per = rows * cfh::NBINS, per_small = rows * SMALL_ANGLE_BINS;
    if (N <= 0) {
        hipLaunchKernelGGL(cfh::zero_outputs_kernel, dim3((per + 255) / 256), dim3(256), 0, st, per, gW_dist, nullptr,
                           nullptr, nullptr);
        hipLaunchKernelGGL(cfh::zero_outputs_kernel, dim3((per_small + 255) / 256), dim3(256), 0, st, per_small, gW_axis1,
                           gW_axis2, gW_axis3, nullptr);
        return finish_launch("zero_outputs");
    }
    const size_t off = padded_offset(p, N);
    if ((rc = check_workspace(workspace, workspace_bytes, off + 6 * (size_t)per * sizeof(float)))) return rc;
    float* padded = reinterpret_cast<float*>(reinterpret_cast<char*>(workspace) + off);
    float* gpad = padded + 3 * per;
    hipLaunchKernelGGL(cfh::pad_bins_kernel, dim3((3 * per + 255) / 256), dim3(256), 0, st, W_axis1, W_axis2, W_axis3, rows,
                       SMALL_ANGLE_BINS, padded);
    cfh_params q = *p;
    q.flags |= CFH_FLAG_SINGLE_STREAM;
    rc = framed_pe_backward_impl(&q, a_ih, rpos, tvecs, rvlen, batch, edges, e_start, order, W_dist, padded, padded + per,
                                 padded + 2 * per, frames, z, gz, gpsi, shat, N, E, B, ga, gW_dist, gpad, gpad + per,
                                 gpad + 2 * per, workspace, workspace_bytes, stream);
    if (rc) return rc;
    hipLaunchKernelGGL(cfh::unpad_bins_kernel, dim3((3 * per_small + 255) / 256), dim3(256), 0, st, gpad, rows,
                       SMALL_ANGLE_BINS, gW_axis1, gW_axis2, gW_axis3);
    return finish_launch("framed_pe_backward (16-bin angle basis)");
}

int cfh_framed_pe_backward_pairwise(const cfh_params* p, const float* a_ih, const float* rpos, const float* tvecs,
                                    const float* rvlen, const int64_t* batch, const int64_t* edges,
                                    const int64_t* e_start, const int32_t* order, const float* frames, const float* z,
                                    const float* gz, const float* g_pair, int64_t N, int64_t E, int64_t B, float* ga,
                                    void* workspace, size_t workspace_bytes, void* stream) {
    if (!g_pair) return fail(CFH_EINVAL, "g_pair must not be NULL");
    if (N <= 0) return check_params(p);
    return framed_pe_backward_impl(p, a_ih, rpos, tvecs, rvlen, batch, edges, e_start, order, nullptr, nullptr, nullptr,
                                   nullptr, frames, z, gz, nullptr, nullptr, N, E, B, ga, nullptr, nullptr, nullptr,
                                   nullptr, workspace, workspace_bytes, stream, g_pair);
}

namespace {
int check_dpa(const void* q, const void* k, const void* v, const int64_t* edges, const int64_t* e_start,
              int64_t N, int64_t H, int64_t Dh, int64_t E) {
    if (N < 0 || E < 0) return fail(CFH_EINVAL, "negative size N=%lld E=%lld", (long long)N, (long long)E);
    if (H < 1 || H > MAX_HEADS) return fail(CFH_EINVAL, "H %lld outside 1..%d", (long long)H, MAX_HEADS);
    if (Dh != cfh::DH) return fail(CFH_EINVAL, "head_dim %lld not compiled (only %d)", (long long)Dh, cfh::DH);
    if (N > 0x7fffffffLL / 64 || E > 0x7fffffffLL / 64)
        return fail(CFH_EINVAL, "N=%lld or E=%lld beyond the 32-bit index range of the kernels", (long long)N, (long long)E);
    if (N > 0 && (!q || !k || !v || !e_start)) return fail(CFH_EINVAL, "q, k, v and e_start must not be NULL");
    if (E > 0 && !edges) return fail(CFH_EINVAL, "edges must not be NULL");
    return CFH_OK;
}
}  // namespace

int cfh_fused_dpa_forward(const float* q, const float* k, const float* v, const float* aij,
                          const float* bij, const int64_t* edges, const int64_t* e_start, int64_t N,
                          int64_t H, int64_t Dh, int64_t E, float* prob, float* out, void* stream) {
    int rc = check_dpa(q, k, v, edges, e_start, N, H, Dh, E);
    if (rc) return rc;
    if (N == 0) return CFH_OK;
    if (!out || (E > 0 && !prob)) return fail(CFH_EINVAL, "prob and out must not be NULL");
    cfh::DpaArgs A;
    std::memset(&A, 0, sizeof(A));
    A.q = q; A.k = k; A.v = v; A.aij = aij; A.bij = bij; A.edges = edges; A.e_start = e_start;
    A.prob = prob; A.out = out; A.N = (int32_t)N; A.H = (int32_t)H; A.E = (int32_t)E;
    const int64_t items = N * H;
    hipLaunchKernelGGL(cfh::dpa_fwd_kernel, dim3((unsigned)((items + cfh::DPA_WAVES - 1) / cfh::DPA_WAVES)),
                       dim3(cfh::WAVE * cfh::DPA_WAVES), 0, (hipStream_t)stream, A);
    return finish_launch("fused_dpa_forward");
}

int cfh_fused_dpa_backward(const float* q, const float* k, const float* v, const float* aij,
                           const float* bij, const int64_t* edges, const int64_t* e_start,
                           const float* prob, const float* out, const float* gout, int64_t N,
                           int64_t H, int64_t Dh, int64_t E, float* gq, float* gk, float* gv,
                           float* gaij, float* gbij, void* stream) {
    int rc = check_dpa(q, k, v, edges, e_start, N, H, Dh, E);
    if (rc) return rc;
    if (N == 0) return CFH_OK;
    if (!out || !gout || !gq || !gk || !gv) return fail(CFH_EINVAL, "out, gout, gq, gk and gv must not be NULL");
    if (E > 0 && (!prob || !gaij)) return fail(CFH_EINVAL, "prob and gaij must not be NULL");
    (void)aij;
    cfh::DpaArgs A;
    std::memset(&A, 0, sizeof(A));
    A.q = q; A.k = k; A.v = v; A.bij = bij; A.edges = edges; A.e_start = e_start;
    A.prob = const_cast<float*>(prob); A.out = const_cast<float*>(out); A.go = gout;
    A.gq = gq; A.gk = gk; A.gv = gv; A.gaij = gaij; A.gbij = gbij;
    A.N = (int32_t)N; A.H = (int32_t)H; A.E = (int32_t)E;
    const int64_t items = N * H;
    const dim3 grid((unsigned)((items + cfh::DPA_WAVES - 1) / cfh::DPA_WAVES)), block(cfh::WAVE * cfh::DPA_WAVES);
    hipLaunchKernelGGL(cfh::dpa_bwd_row_kernel, grid, block, 0, (hipStream_t)stream, A);
    hipLaunchKernelGGL(cfh::dpa_bwd_col_kernel, grid, block, 0, (hipStream_t)stream, A);
    return finish_launch("fused_dpa_backward");
}

int cfh_pair_layout_check(const int64_t* edges, const int64_t* e_start, int64_t N, int64_t E,
                          int32_t* flag, void* stream) {
    if (!flag) return fail(CFH_EINVAL, "flag must not be NULL");
    if (N < 0 || E < 0 || N > 0x7fffffffLL / 64 || E > 0x7fffffffLL / 64)
        return fail(CFH_EINVAL, "N=%lld or E=%lld outside the index range of the kernels", (long long)N, (long long)E);
    if (N > 0 && (!e_start || (E > 0 && !edges))) return fail(CFH_EINVAL, "edges and e_start must not be NULL");
    hipLaunchKernelGGL(cfh::set_flag_kernel, dim3(1), dim3(1), 0, (hipStream_t)stream, flag, 0);
    if (N > 0)
        hipLaunchKernelGGL(cfh::dpa_check_layout_kernel, dim3((unsigned)((N + 255) / 256)), dim3(256), 0,
                           (hipStream_t)stream, edges, e_start, (int)N, (int)E, flag);
    return finish_launch("pair_layout_check");
}

int cfh_crystal_mean_forward(const float* x, const int64_t* atom_start, int64_t N, int64_t B,
                             int64_t C, float* out, void* stream) {
    if (N < 0 || B < 0 || C < 0 || C > 0x7fffffffLL || N > 0x7fffffffLL || B > 0x7fffffffLL)
        return fail(CFH_EINVAL, "sizes N=%lld B=%lld C=%lld out of range", (long long)N, (long long)B, (long long)C);
    if (B == 0 || C == 0) return CFH_OK;
    if (!atom_start || !out || (N > 0 && !x)) return fail(CFH_EINVAL, "x, atom_start and out must not be NULL");
    if (C % 4 == 0 && C <= 1024 && ((uintptr_t)x & 15) == 0 && ((uintptr_t)out & 15) == 0) {
        hipLaunchKernelGGL(cfh::crystal_mean_fwd_vec_kernel, dim3((unsigned)B), dim3(256), 0, (hipStream_t)stream, x,
                           atom_start, (int)B, (int)C, out);
        return finish_launch("crystal_mean_forward");
    }
    const int threads = C >= 256 ? 256 : (C >= 128 ? 128 : 64);
    hipLaunchKernelGGL(cfh::crystal_mean_fwd_kernel, dim3((unsigned)B), dim3(threads), 0, (hipStream_t)stream, x,
                       atom_start, (int)B, (int)C, out);
    return finish_launch("crystal_mean_forward");
}

int cfh_crystal_mean_backward(const float* gout, const int64_t* batch, const int64_t* atom_start,
                              int64_t N, int64_t B, int64_t C, float* gx, void* stream) {
    if (N < 0 || B < 0 || C < 0 || C > 0x7fffffffLL || N > 0x7fffffffLL || B > 0x7fffffffLL)
        return fail(CFH_EINVAL, "sizes N=%lld B=%lld C=%lld out of range", (long long)N, (long long)B, (long long)C);
    if (N == 0 || C == 0) return CFH_OK;
    if (!gout || !batch || !atom_start || !gx) return fail(CFH_EINVAL, "gout, batch, atom_start and gx must not be NULL");
    const size_t total = (size_t)N * (size_t)C;
    hipLaunchKernelGGL(cfh::crystal_mean_bwd_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0,
                       (hipStream_t)stream, gout, batch, atom_start, (int)N, (int)C, gx);
    return finish_launch("crystal_mean_backward");
}

int cfh_linear_weight_bias_grad(const float* x, const float* dy, int64_t N, int64_t I, int64_t O,
                                float* dW, float* db, void* stream) {
    if (N < 0 || I < 1 || O < 1 || N > 0x7fffffffLL / 64 || I > 65536 || O > 65536)
        return fail(CFH_EINVAL, "sizes N=%lld I=%lld O=%lld out of range", (long long)N, (long long)I, (long long)O);
    if (!dW || (N > 0 && (!x || !dy))) return fail(CFH_EINVAL, "x, dy and dW must not be NULL");
    hipStream_t st = (hipStream_t)stream;
    const int nw = (int)(O * I), nb = (int)O;
    hipLaunchKernelGGL(cfh::zero2_kernel, dim3((nw + 255) / 256), dim3(256), 0, st, dW, nw, db, nb);
    if (N > 0) {
        const int bx = (int)((I + 63) / 64), by = (int)((O + 63) / 64);
        int slices = (512 + bx * by - 1) / (bx * by);      // about 512 workgroups of 4 wavefronts
        const int max_slices = (int)((N + 31) / 32);
        if (slices > max_slices) slices = max_slices;
        if (slices < 1) slices = 1;
        int rows = (int)((N + slices - 1) / slices);
        rows = (rows + 3) & ~3;
        slices = (int)((N + rows - 1) / rows);
        hipLaunchKernelGGL(cfh::linear_wgrad_kernel, dim3(bx, by, slices), dim3(256), 0, st, x, dy, (int)N, (int)I,
                           (int)O, rows, dW, db);
    }
    return finish_launch("linear_weight_bias_grad");
}

static int attention_inputs_args(cfh::AttnInArgs& A, const float* qkv, const float* w, const float* gauss, float c1,
                                 float lb, float c2, float q_scale, int64_t N, int32_t H, int32_t Dh) {
    if (Dh != 16 || H < 1 || 256 % (H * Dh) != 0)
        return fail(CFH_EINVAL, "attention inputs: head_dim must be 16 and 256 a multiple of H*Dh (H=%d Dh=%d)", H, Dh);
    if (N < 0 || N > 0x7fffffffLL / (3 * H * Dh)) return fail(CFH_EINVAL, "N=%lld out of range", (long long)N);
    if (N > 0 && (!qkv || !w)) return fail(CFH_EINVAL, "qkv and lattice_w must not be NULL");
    A = cfh::AttnInArgs{};
    A.qkv = qkv; A.w = w; A.gauss = gauss; A.N = (int)N; A.HD = H * Dh;
    A.c1 = c1; A.lb = lb; A.c2 = c2; A.q_scale = q_scale;
    return CFH_OK;
}

int cfh_attention_inputs_forward(const float* qkv, const float* lattice_w, const float* gauss_scale_dev,
                                 float c1, float lb, float c2, float q_scale, int64_t N, int32_t H, int32_t Dh,
                                 float* qs, float* k, float* v, float* a, void* stream) {
    cfh::AttnInArgs A;
    if (int rc = attention_inputs_args(A, qkv, lattice_w, gauss_scale_dev, c1, lb, c2, q_scale, N, H, Dh)) return rc;
    if (N == 0) return CFH_OK;
    if (!qs || !k || !v || !a) return fail(CFH_EINVAL, "qs, k, v and a must not be NULL");
    A.qs = qs; A.k = k; A.v = v; A.a = a;
    const long total = (long)N * A.HD;
    hipLaunchKernelGGL(cfh::attention_inputs_fwd_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0,
                       (hipStream_t)stream, A);
    return finish_launch("attention_inputs_forward");
}

int cfh_attention_inputs_backward(const float* qkv, const float* lattice_w, const float* gauss_scale_dev,
                                  float c1, float lb, float c2, float q_scale, const float* gqs, const float* gk,
                                  const float* gv, const float* ga, int64_t N, int32_t H, int32_t Dh,
                                  float* gqkv, float* g_lattice_w, void* workspace, size_t workspace_bytes,
                                  void* stream) {
    cfh::AttnInArgs A;
    if (int rc = attention_inputs_args(A, qkv, lattice_w, gauss_scale_dev, c1, lb, c2, q_scale, N, H, Dh)) return rc;
    if (N > 0 && !gqkv) return fail(CFH_EINVAL, "gqkv must not be NULL");
    hipStream_t st = (hipStream_t)stream;
    A.rows_per_block = 4 * (256 / A.HD);
    const int blocks = (int)((N + A.rows_per_block - 1) / A.rows_per_block);
    if (int rc = check_workspace(workspace, workspace_bytes, (size_t)blocks * A.HD * sizeof(float))) return rc;
    if (N > 0) {
        A.gqs = gqs; A.gk = gk; A.gv = gv; A.ga = ga; A.gqkv = gqkv; A.gw = g_lattice_w;
        A.partial = (float*)workspace;
        hipLaunchKernelGGL(cfh::attention_inputs_bwd_kernel, dim3((unsigned)blocks), dim3(256), 0, st, A);
    }
    if (g_lattice_w)
        hipLaunchKernelGGL(cfh::attention_inputs_gw_kernel, dim3((A.HD + 31) / 32), dim3(1024), 0, st,
                           (const float*)workspace, blocks, A.HD, g_lattice_w);
    return finish_launch("attention_inputs_backward");
}

}  // extern "C"
namespace {
int check_wgrad_jobs(const cfh_linear_grad_job* jobs, int32_t njobs) {
    if (njobs < 0 || (njobs > 0 && !jobs)) return fail(CFH_EINVAL, "jobs is NULL or njobs negative");
    for (int32_t j = 0; j < njobs; j++) {
        const cfh_linear_grad_job& J = jobs[j];
        if (J.N < 0 || J.I < 1 || J.O < 1 || J.N > 0x7fffffffLL / 64 || J.I > 65536 || J.O > 65536 || J.ldx < J.I ||
            J.ldy < J.O || J.ldx > (1LL << 26) || J.ldy > (1LL << 26))
            return fail(CFH_EINVAL, "job %d: sizes N=%lld I=%lld O=%lld ldx=%lld ldy=%lld out of range", (int)j,
                        (long long)J.N, (long long)J.I, (long long)J.O, (long long)J.ldx, (long long)J.ldy);
        if ((!J.dW && !J.db) || (J.N > 0 && (!J.dy || (J.dW && !J.x))))
            return fail(CFH_EINVAL, "job %d: dy, one of dW and db, and x with dW must not be NULL", (int)j);
    }
    return CFH_OK;
}
// The launch of the jobs [first, last): slices and workgroup numbers of every job; returns the number of tiles that
// several slices share.
int plan_wgrad(const cfh_linear_grad_job* jobs, int32_t first, int32_t last, cfh::WgradJobs& T) {
    // a job whose shape and alignment allow it takes the variant with 16-byte loads
    auto wide = [](const cfh_linear_grad_job& J) {
        return J.dW && J.O % 64 == 0 && J.I % 64 == 0 && J.ldx % 4 == 0 && J.ldy % 4 == 0 &&
               ((uintptr_t)J.x | (uintptr_t)J.dy) % 16 == 0;
    };
    auto tiles_of = [&](const cfh_linear_grad_job& J, long& bx, long& by) {
        bx = J.dW ? (J.I + 63) / 64 : 1;
        by = (J.O + 63) / 64;
    };
    long tiles = 0;
    for (int32_t j = first; j < last; j++)
        if (jobs[j].N > 0) {
            long bx, by;
            tiles_of(jobs[j], bx, by);
            tiles += bx * by;
        }
    T = cfh::WgradJobs{};
    if (tiles == 0) return 0;
    // slices of a job: the workgroups stay just below the four per compute unit that are resident at once (a few
    // more would run as a second round and double the time)
    int cus = device_cus();
    if (cus <= 0) cus = 256;
    const long target = 4L * cus - 24;
    const int want = (int)(target / tiles > 0 ? target / tiles : 1);
    int blocks = 0, tile0 = 0;
    for (int32_t j = first; j < last; j++) {
        const cfh_linear_grad_job& J = jobs[j];
        if (J.N == 0) continue;
        cfh::WgradJob& W = T.job[T.njobs++];
        W.x = J.x; W.dy = J.dy; W.dW = J.dW; W.db = J.db;
        W.N = (int)J.N; W.I = (int)J.I; W.O = (int)J.O; W.ldx = (int)J.ldx; W.ldy = (int)J.ldy;
        long bx, by;
        tiles_of(J, bx, by);
        W.bx = (int)bx; W.by = (int)by; W.wide = wide(J) ? 1 : 0;
        int slices = want;
        const int max_slices = (int)((J.N + 31) / 32);
        if (slices > max_slices) slices = max_slices;
        if (slices < 1) slices = 1;
        int rows = (int)((J.N + slices - 1) / slices);
        rows = (rows + 3) & ~3;
        slices = (int)((J.N + rows - 1) / rows);
        W.rows_per_slice = rows;
        W.slices = slices;
        W.block0 = blocks;
        W.tile0 = tile0;
        blocks += W.bx * W.by * slices;
        if (slices > 1) tile0 += W.bx * W.by;
    }
    T.blocks = blocks;
    T.split_tiles = tile0;
    return tile0;
}
// Order of the jobs of a call and where one launch ends and the next begins.  With float atomics: the caller's
// order, 32 jobs a launch.  For sums in a fixed order two jobs that add to the same memory (a weight used twice in
// one pass) must not share a launch -- the sums reach the outputs without atomics -- so a job goes
// to the launch after the last one that holds a job whose dW or db overlaps its own.
void wgrad_launches(const cfh_linear_grad_job* jobs, int32_t njobs, bool fixed_order,
                    std::vector<cfh_linear_grad_job>& ordered, std::vector<int32_t>& ends) {
    std::vector<int> round(njobs, 0);
    int rounds = 1;
    if (fixed_order) {
        auto overlap = [](const float* a, size_t na, const float* b, size_t nb) {
            return a && b && (uintptr_t)a < (uintptr_t)(b + nb) && (uintptr_t)b < (uintptr_t)(a + na);
        };
        for (int32_t j = 1; j < njobs; j++)
            for (int32_t i = 0; i < j; i++) {
                const cfh_linear_grad_job &A = jobs[i], &B = jobs[j];
                if (round[i] >= round[j] &&
                    (overlap(A.dW, (size_t)A.O * A.I, B.dW, (size_t)B.O * B.I) || overlap(A.db, A.O, B.db, B.O)))
                    round[j] = round[i] + 1;
            }
        for (int32_t j = 0; j < njobs; j++) rounds = round[j] + 1 > rounds ? round[j] + 1 : rounds;
    }
    ordered.clear();
    ends.clear();
    for (int r = 0; r < rounds; r++) {
        int in_launch = 0;
        for (int32_t j = 0; j < njobs; j++) {
            if (round[j] != r) continue;
            if (in_launch == cfh::WGRAD_MAX_JOBS) { ends.push_back((int32_t)ordered.size()); in_launch = 0; }
            ordered.push_back(jobs[j]);
            in_launch++;
        }
        if (in_launch) ends.push_back((int32_t)ordered.size());
    }
}
}  // namespace
extern "C" {

size_t cfh_linear_weight_bias_grad_batch_workspace_bytes(const cfh_linear_grad_job* jobs, int32_t njobs) {
    if (check_wgrad_jobs(jobs, njobs) != CFH_OK) return 0;
    std::vector<cfh_linear_grad_job> ordered;
    std::vector<int32_t> ends;
    wgrad_launches(jobs, njobs, true, ordered, ends);
    size_t need = 256;
    int32_t first = 0;
    for (int32_t last : ends) {
        cfh::WgradJobs T;
        plan_wgrad(ordered.data(), first, last, T);
        const size_t bytes = (size_t)T.blocks * cfh::WG_PART * sizeof(float);
        if (bytes > need) need = bytes;
        first = last;
    }
    return need;
}

int cfh_linear_weight_bias_grad_batch(const cfh_linear_grad_job* jobs, int32_t njobs, void* workspace,
                                      size_t workspace_bytes, void* stream) {
    int rc = check_wgrad_jobs(jobs, njobs);
    if (rc) return rc;
    hipStream_t st = (hipStream_t)stream;
    std::vector<cfh_linear_grad_job> ordered;
    std::vector<int32_t> ends;
    wgrad_launches(jobs, njobs, workspace != nullptr, ordered, ends);
    int32_t first = 0;
    for (int32_t last : ends) {
        cfh::WgradJobs T;
        plan_wgrad(ordered.data(), first, last, T);
        first = last;
        if (T.blocks == 0) continue;
        if (workspace) {
            // scratch for the sums in a fixed order: a stored tile per workgroup; the launches of one call run one
            // after the other and share it
            if ((rc = check_workspace(workspace, workspace_bytes, (size_t)T.blocks * cfh::WG_PART * sizeof(float))))
                return rc;
            T.scratch.partials = reinterpret_cast<float*>(workspace);
        }
        hipLaunchKernelGGL(cfh::linear_wgrad_batch_kernel, dim3((T.blocks + 7) & ~7), dim3(256), 0, st, T);
        if (workspace && T.split_tiles > 0)
            hipLaunchKernelGGL(cfh::linear_wgrad_sum_kernel, dim3(4 * T.split_tiles), dim3(256), 0, st, T);
    }
    return finish_launch("linear_weight_bias_grad_batch");
}

int cfh_layer_bridge_forward(const float* attn, const float* x_res, int64_t N, int32_t D, int32_t F, const float* Wo,
                             const float* bo, const float* W1, const float* b1, const float* W2, const float* b2,
                             const float* Wqkv, const float* bqkv, const float* lattice_w,
                             const float* gauss_scale_dev, float c1, float lb, float c2, float q_scale, int32_t H,
                             float* x1, float* h, float* x2, float* qkv, float* qs, float* k, float* v, float* a,
                             void* stream) {
    if (N < 0 || N > 0x7fffffffLL / 1024 || D < 128 || F < 128 || D % 128 != 0 || F % 128 != 0 || D > 65536 || F > 65536)
        return fail(CFH_EINVAL, "layer bridge: N=%lld, D=%d and F=%d must be multiples of 128", (long long)N, (int)D, (int)F);
    if (H < 1 || H * cfh::DH != D || cfh::BR_ROWS * H > 64 * cfh::BR_WAVES)
        return fail(CFH_EINVAL, "layer bridge: D=%d must be 16 x H=%d, H at most %d", (int)D, (int)H, 64 * cfh::BR_WAVES / cfh::BR_ROWS);
    if (N == 0) return CFH_OK;
    if (!attn || !x_res || !Wo || !W1 || !W2 || !x1 || !h || !x2)
        return fail(CFH_EINVAL, "layer bridge: attn, x_res, the weights and x1, h, x2 must not be NULL");
    if (Wqkv && (!lattice_w || !qkv || !qs || !k || !v || !a))
        return fail(CFH_EINVAL, "layer bridge: with Wqkv, lattice_w and qkv, qs, k, v, a must not be NULL");
    const int wide = F > 3 * D ? F : 3 * D;
    const size_t lds = ((size_t)cfh::BR_ROWS * (2 * (D + cfh::BR_PAD) + wide + cfh::BR_PAD) +
                        (size_t)cfh::BR_WAVES * cfh::BR_STAGE_FLOATS) * sizeof(float);
    if (lds > 160 * 1024) return fail(CFH_EINVAL, "layer bridge: D=%d, F=%d need %zu bytes of LDS", (int)D, (int)F, lds);
    static int lds_set[64] = {0};
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return fail(CFH_ELAUNCH, "layer bridge: no current device");
    if (lds_set[dev] < (int)lds) {
        if (hipFuncSetAttribute((const void*)cfh::layer_bridge_fwd_kernel, hipFuncAttributeMaxDynamicSharedMemorySize,
                                (int)lds) != hipSuccess)
            return fail(CFH_ELAUNCH, "layer bridge: %zu bytes of LDS refused", lds);
        lds_set[dev] = (int)lds;
    }
    cfh::BridgeArgs A{};
    A.attn = attn; A.xres = x_res; A.Wo = Wo; A.bo = bo; A.W1 = W1; A.b1 = b1; A.W2 = W2; A.b2 = b2;
    A.Wq = Wqkv; A.bq = bqkv; A.lattice_w = lattice_w; A.gauss = gauss_scale_dev;
    A.x1 = x1; A.h = h; A.x2 = x2; A.qkv = qkv; A.qs = qs; A.k = k; A.v = v; A.a = a;
    A.N = (int)N; A.D = D; A.F = F; A.H = H;
    A.c1 = c1; A.lb = lb; A.c2 = c2; A.q_scale = q_scale;
    hipLaunchKernelGGL(cfh::layer_bridge_fwd_kernel, dim3((unsigned)((N + cfh::BR_ROWS - 1) / cfh::BR_ROWS)),
                       dim3(64 * cfh::BR_WAVES), lds, (hipStream_t)stream, A);
    return finish_launch("layer_bridge_forward");
}

int cfh_layer_bridge_backward(const float* g_x2, const float* gqkv, const float* h, const float* Wqkv,
                              const float* W2, const float* W1, const float* Wo, int64_t N, int32_t D, int32_t F,
                              float* g2, float* gh, float* g1, float* g_attn, const cfh_attention_inputs_grad* ai,
                              void* stream) {
    if (N < 0 || N > 0x7fffffffLL / 1024 || D < 128 || F < 128 || D % 128 != 0 || F % 128 != 0 || D > 65536 || F > 65536)
        return fail(CFH_EINVAL, "layer bridge: N=%lld, D=%d and F=%d must be multiples of 128", (long long)N, (int)D, (int)F);
    if (N == 0) return CFH_OK;
    if (!h || !W2 || !W1 || !Wo || !gh || !g1 || !g_attn || ((gqkv || ai) && (!Wqkv || !g2)))
        return fail(CFH_EINVAL, "layer bridge backward: h, the weights and gh, g1, g_attn (with gqkv: Wqkv and g2) must not be NULL");
    if (ai && (gqkv || !ai->qkv || !ai->lattice_w || !ai->gqkv || !ai->gw_partial || ai->H < 1 || ai->H * cfh::DH != D ||
               cfh::BR_ROWS * ai->H > 64 * cfh::BR_WAVES))
        return fail(CFH_EINVAL, "layer bridge backward: attention-input gradients need qkv, lattice_w, gqkv, gw_partial, "
                                "D = 16 H, and no gqkv argument");
    const size_t lds = cfh::bridge_bwd_lds_floats(D, F) * sizeof(float);
    if (lds > 160 * 1024) return fail(CFH_EINVAL, "layer bridge backward: D=%d, F=%d need %zu bytes of LDS", (int)D, (int)F, lds);
    static int lds_set[64] = {0};
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return fail(CFH_ELAUNCH, "layer bridge: no current device");
    if (lds_set[dev] < (int)lds) {
        if (hipFuncSetAttribute((const void*)cfh::layer_bridge_bwd_kernel, hipFuncAttributeMaxDynamicSharedMemorySize,
                                (int)lds) != hipSuccess)
            return fail(CFH_ELAUNCH, "layer bridge backward: %zu bytes of LDS refused", lds);
        lds_set[dev] = (int)lds;
    }
    cfh::BridgeBwdArgs A{};
    A.g_x2 = g_x2; A.gqkv = gqkv; A.h = h; A.Wq = Wqkv; A.W2 = W2; A.W1 = W1; A.Wo = Wo;
    A.g2 = g2; A.gh = gh; A.g1 = g1; A.g_attn = g_attn;
    A.N = (int)N; A.D = D; A.F = F;
    if (ai) {
        A.ai_qkv = ai->qkv; A.ai_w = ai->lattice_w; A.ai_gauss = ai->gauss_scale_dev;
        A.ai_gqs = ai->gqs; A.ai_gk = ai->gk; A.ai_gv = ai->gv; A.ai_ga = ai->ga;
        A.gqkv_out = ai->gqkv; A.gw_partial = ai->gw_partial; A.H = ai->H;
        A.c1 = ai->c1; A.lb = ai->lb; A.c2 = ai->c2; A.q_scale = ai->q_scale;
    }
    hipLaunchKernelGGL(cfh::layer_bridge_bwd_kernel, dim3((unsigned)((N + cfh::BR_ROWS - 1) / cfh::BR_ROWS)),
                       dim3(64 * cfh::BR_WAVES), lds, (hipStream_t)stream, A);
    return finish_launch("layer_bridge_backward");
}

int cfh_crystal_geometry(const float* pos, const int64_t* batch, const float* tvecs, const int64_t* sizes,
                         int64_t N, int64_t B, int64_t E, int64_t* edges, float* rpos, float* recip,
                         float* rvlen, float* vcell, int64_t* e_start, int64_t* atom_start, int32_t* order,
                         void* workspace, size_t workspace_bytes, void* stream) {
    if (N < 0 || B < 0 || E < 0 || N > 0x7fffffffLL / 64 || B > 0x7fffffffLL / 64)
        return fail(CFH_EINVAL, "sizes N=%lld B=%lld E=%lld out of range", (long long)N, (long long)B, (long long)E);
    if (!e_start || !atom_start || (B > 0 && (!tvecs || !sizes || !recip || !rvlen || !vcell)) ||
        (N > 0 && (!pos || !batch || !order)) || (E > 0 && (!edges || !rpos)))
        return fail(CFH_EINVAL, "geometry: an input or output pointer is NULL");
    if (int rc = check_workspace(workspace, workspace_bytes, (size_t)(2 * B + 1) * sizeof(int64_t))) return rc;
    cfh::GeometryArgs A{};
    A.pos = pos; A.batch = batch; A.tvecs = tvecs; A.sizes = sizes;
    A.edges = edges; A.rpos = rpos; A.recip = recip; A.rvlen = rvlen; A.vcell = vcell;
    A.e_start = e_start; A.order = order; A.atom_start = atom_start;
    A.pair_start = reinterpret_cast<int64_t*>(workspace);
    A.order_start = A.pair_start + (B + 1);
    A.N = (int32_t)N; A.B = (int32_t)B; A.E = E;
    hipStream_t st = (hipStream_t)stream;
    hipLaunchKernelGGL(cfh::geometry_crystals_kernel, dim3(2), dim3(cfh::GEO_THREADS), 0, st, A);
    hipLaunchKernelGGL(cfh::geometry_atoms_kernel, dim3((unsigned)((N + 256) / 256)), dim3(256), 0, st, A);
    if (E > 0)
        hipLaunchKernelGGL(cfh::geometry_pairs_kernel, dim3((unsigned)((E + 255) / 256)), dim3(256), 0, st, A);
    return finish_launch("crystal_geometry");
}

int cfh_small_linear_forward(const float* x, const float* W, const float* b, int64_t M, int64_t N, int64_t K,
                             int32_t relu, float* y, void* stream) {
    if (M < 0 || N < 1 || K < 16 || K % 16 != 0 || M > 0x7fffffffLL / 64 || N > 65536 || K > 65536)
        return fail(CFH_EINVAL, "small linear forward: M=%lld N=%lld K=%lld (K must be a multiple of 16)", (long long)M,
                    (long long)N, (long long)K);
    if (M == 0) return CFH_OK;
    if (!x || !W || !y || (((uintptr_t)x | (uintptr_t)W) & 15)) return fail(CFH_EINVAL, "x, W, y must not be NULL; x, W 16-byte aligned");
    hipLaunchKernelGGL(cfh::small_linear_fwd_kernel, dim3((unsigned)((M + 63) / 64), (unsigned)((N + 63) / 64)), dim3(256), 0,
                       (hipStream_t)stream, x, W, b, y, (int)M, (int)N, (int)K, (int)relu);
    return finish_launch("small_linear_forward");
}

int cfh_small_linear_dx(const float* dy, const float* W, int64_t M, int64_t N, int64_t K, float* dx, void* stream) {
    if (M < 0 || K < 1 || N < 1 || M > 0x7fffffffLL / 64 || N > 65536 || K > 65536)
        return fail(CFH_EINVAL, "small linear dx: M=%lld N=%lld K=%lld out of range", (long long)M, (long long)N, (long long)K);
    if (M == 0) return CFH_OK;
    if (!dy || !W || !dx) return fail(CFH_EINVAL, "dy, W, dx must not be NULL");
    if (N % 16 != 0 || ((uintptr_t)dy & 15)) {
        if (N > 64) return fail(CFH_EINVAL, "small linear dx: N=%lld must be a multiple of 16 (with dy 16-byte aligned) or at most 64", (long long)N);
        hipLaunchKernelGGL(cfh::small_linear_dx_narrow_kernel, dim3((unsigned)((M * K + 255) / 256)), dim3(256), 0,
                           (hipStream_t)stream, dy, W, dx, (int)M, (int)N, (int)K);
        return finish_launch("small_linear_dx");
    }
    hipLaunchKernelGGL(cfh::small_linear_dx_kernel, dim3((unsigned)((M + 63) / 64), (unsigned)((K + 63) / 64)), dim3(256), 0,
                       (hipStream_t)stream, dy, W, dx, (int)M, (int)N, (int)K);
    return finish_launch("small_linear_dx");
}

int cfh_adamw_step_batch(const cfh_adamw_job* jobs, int32_t njobs, float lr, float beta1, float beta2, float eps,
                         float weight_decay, uint64_t* step_dev, void* stream) {
    if (njobs < 0 || (njobs > 0 && !jobs)) return fail(CFH_EINVAL, "jobs is NULL or njobs negative");
    if (!step_dev) return fail(CFH_EINVAL, "step_dev must not be NULL");
    if (!(beta1 >= 0.0f && beta1 < 1.0f && beta2 >= 0.0f && beta2 < 1.0f && eps >= 0.0f))
        return fail(CFH_EINVAL, "adamw: beta1 = %g, beta2 = %g must lie in [0, 1), eps = %g must not be negative", beta1, beta2, eps);
    for (int32_t j = 0; j < njobs; j++) {
        const cfh_adamw_job& J = jobs[j];
        if (J.n < 0 || J.n > 0x7fffffffLL - cfh::ADAMW_BLOCK_ELEMS)
            return fail(CFH_EINVAL, "adamw job %d: n = %lld out of range", (int)j, (long long)J.n);
        if (J.n > 0 && (!J.param || !J.grad || !J.exp_avg || !J.exp_avg_sq))
            return fail(CFH_EINVAL, "adamw job %d: param, grad, exp_avg, exp_avg_sq must not be NULL", (int)j);
    }
    hipStream_t st = (hipStream_t)stream;
    int32_t j = 0;
    while (j < njobs) {
        cfh::AdamWJobs T{};
        T.lr = lr; T.beta1 = beta1; T.beta2 = beta2; T.eps = eps; T.wd = weight_decay;
        T.step = reinterpret_cast<const unsigned long long*>(step_dev);
        long blocks = 0;
        for (; j < njobs && T.njobs < cfh::ADAMW_MAX_JOBS; j++) {
            if (jobs[j].n == 0) continue;
            const long nb = (long)((jobs[j].n + cfh::ADAMW_BLOCK_ELEMS - 1) / cfh::ADAMW_BLOCK_ELEMS);
            if (blocks + nb > 0x7fffffffL) break;
            cfh::AdamWJob& W = T.job[T.njobs++];
            W.p = jobs[j].param; W.g = jobs[j].grad; W.m = jobs[j].exp_avg; W.v = jobs[j].exp_avg_sq;
            W.n = (int)jobs[j].n; W.block0 = (int)blocks;
            blocks += nb;
        }
        if (T.njobs == 0) break;
        hipLaunchKernelGGL(cfh::adamw_batch_kernel, dim3((unsigned)blocks), dim3(256), 0, st, T);
    }
    hipLaunchKernelGGL(cfh::adamw_advance_kernel, dim3(1), dim3(1), 0, st, reinterpret_cast<unsigned long long*>(step_dev));
    return finish_launch("adamw_step_batch");
}

}  // extern "C"

// ---- fused attention core ----------------------------------------------------------------------------------------
namespace {
struct CoreLayout {
    size_t items, sorted, near, wcat, gwcat, G, slow, total;
    int hw;
    int prep_blocks;      // blocks of 256 threads of the launch that makes the item records
};
size_t align256(size_t x) { return (x + 255) & ~(size_t)255; }
CoreLayout core_layout(const cfh_params* p, int64_t N, int64_t E, int64_t B, bool backward) {
    CoreLayout L;
    L.hw = cfh::core_hist_words(p->angle_bins);
    size_t off = COUNTER_BYTES;
    L.items = off; off += items_bytes(N > 0 ? N : 1, p->num_heads);
    L.sorted = off; off += align256((size_t)(B > 0 ? B : 1) * cfh::FC_TCAP * sizeof(float4));
    L.near = off; if (!backward) off += align256((size_t)(E > 0 ? E : 1) * sizeof(float2));
    L.wcat = off; off += align256((size_t)p->num_heads * cfh::DH * L.hw * sizeof(float));
    L.gwcat = off; if (backward) off += align256((size_t)cfh::CORE_GW_SLICES * p->num_heads * cfh::DH * L.hw * sizeof(float));
    L.G = off; if (backward) off += align256((size_t)(N > 0 ? N : 1) * p->num_heads * L.hw * sizeof(float));
    {
        const int64_t threads = N * p->num_heads > (int64_t)p->num_heads * cfh::NQUEUE ? N * p->num_heads
                                                                                       : (int64_t)p->num_heads * cfh::NQUEUE;
        L.prep_blocks = (int)((threads + 255) / 256);
    }
    // the lists of the records that the main kernel takes first (forward: made with the records)
    // (backward: made by the kernel that writes G, one list per 16 atoms)
    // (a count per list and a slot per record: forward a list per block of records, backward per SLOW_GB_BLOCKS x 16 atoms)
    L.slow = off;
    off += align256(((size_t)(backward ? (N + 15) / 16 + 1 : L.prep_blocks) +
                     (size_t)(backward ? ((N + 15) / 16 + cfh::SLOW_GB_BLOCKS) * 16 * p->num_heads
                                       : (int64_t)L.prep_blocks * cfh::SLOW_PREP_SLOTS)) * sizeof(int32_t));
    L.total = off;
    return L;
}
int check_core_params(const cfh_params* p) {
    int rc = check_params(p);
    if (rc) return rc;
    if (p->dist_bins != cfh::NBINS) return fail(CFH_EINVAL, "fused core: dist_bins must be %d", cfh::NBINS);
    if (!(p->dist_wscale > 0.0f)) return fail(CFH_EINVAL, "fused core: dist_wscale %g must be positive", (double)p->dist_wscale);
    if (p->grad_coef_quirk) return fail(CFH_EINVAL, "fused core: grad_coef_quirk is not available (exact gradients only)");
    if (p->angle_bins == cfh::NBINS && p->angle_wscale < 3.0f)
        return fail(CFH_EINVAL, "fused core: angle_wscale %g < 3 with 64 angle bins: the moment expansion of the angle "
                    "basis (5 terms) is not accurate enough; use the two-step operators", (double)p->angle_wscale);
    if (p->angle_bins == cfh::SMALL_A && p->angle_wscale < 1.0f)
        return fail(CFH_EINVAL, "fused core: angle_wscale %g < 1 with 16 angle bins is not compiled", (double)p->angle_wscale);
    return CFH_OK;
}
// The main kernels address q, k, v, rpos, z and the probabilities with 32-bit byte offsets.
int check_core_sizes(const cfh_params* p, int64_t N, int64_t E) {
    const int64_t lim = (int64_t)1 << 30;      // elements of 4 bytes
    if (N * p->num_heads * cfh::DH >= lim || E * p->num_heads >= lim || E * 3 >= lim)
        return fail(CFH_EINVAL, "fused core: N = %lld atoms or E = %lld pairs beyond the 32-bit offsets of its kernels "
                    "(N x heads x 16 and E x heads must stay below 2^30)", (long long)N, (long long)E);
    return CFH_OK;
}
// the kernels' launch-wide arguments that both directions share; buffers of the caller's cache replace the
// workspace regions of the same content
struct CoreBuffers {
    float4* table;       // sorted shifts (null: not used by this launch)
    float2* near;        // nearest images per pair (forward only; made with the table)
    bool table_ready;
    float* wcat;
    bool wcat_ready;
    bool records_ready;
};
CoreBuffers fill_core(cfh::CoreArgs& C, const cfh_params* p, const CoreLayout& L, const float* qs, const float* k,
                      const float* v, bool has_rvlen, const cfh_core_cache* cache, void* workspace) {
    char* ws = reinterpret_cast<char*>(workspace);
    C.qs = qs; C.k = k; C.v = v;
    const bool adaptive = has_rvlen && p->cutoff_radius != 0.0f;
    const int R0 = adaptive ? p->minimum_range : p->lattice_range;
    const bool tables = R0 >= 1 && (2 * R0 + 1) * (2 * R0 + 1) * (2 * R0 + 1) <= cfh::FC_TCAP;
    CoreBuffers b;
    b.table = nullptr; b.near = nullptr; b.table_ready = false;
    if (tables) {
        const bool own = cache && cache->shift_table;
        b.table = own ? reinterpret_cast<float4*>(cache->shift_table) : reinterpret_cast<float4*>(ws + L.sorted);
        b.table_ready = own && cache->shift_table_ready != 0;
        // the per-pair minima travel with the table: the caller's when it keeps both, else (forward) the workspace's
        if (own && cache->pair_near) b.near = reinterpret_cast<float2*>(cache->pair_near);
        else if (!own && L.near != L.wcat) b.near = reinterpret_cast<float2*>(ws + L.near);
    }
    b.wcat = (cache && cache->wcat) ? cache->wcat : reinterpret_cast<float*>(ws + L.wcat);
    b.wcat_ready = cache && cache->wcat && cache->wcat_ready != 0;
    b.records_ready = cache && cache->records && cache->records_ready != 0;
    if (cache && cache->records) C.K.items = cache->records;
    C.sorted_tab = b.table;
    C.table_R = tables ? R0 : 0;
    C.skip_log2 = p->prune_log2 > 0.0f ? (p->prune_log2 + 8.0f > 32.0f ? p->prune_log2 + 8.0f : 32.0f) : 0.0f;
    return b;
}
// Leading wavefronts of a main kernel, one per listed slow record (the host does not know how many are listed): a
// sixteenth of the records, at least 256.  Listed records beyond that are taken in place like the unlisted.
int slow_wave_count(int64_t N, int H) {
    const int64_t w = (N * H / 16 + 7) / 8 * 8;
    return (int)(w < 256 ? 256 : w);
}
// one wavefront (= workgroup) per (item, head); the hardware deals them to the compute units as slots free up
template <typename Kern>
int launch_core(Kern kern, const cfh::CoreArgs& C, hipStream_t st, const char* what, unsigned waves = 0) {
    if (waves == 0) waves = (unsigned)C.K.N * (unsigned)C.K.H + (unsigned)C.slow_wgs;
    const unsigned blocks = (waves + cfh::CORE_WPB - 1) / cfh::CORE_WPB;
    {
        TimedScope timed(what, st);
        hipLaunchKernelGGL(kern, dim3(blocks), dim3(cfh::WAVE * cfh::CORE_WPB), 0, st, C);
    }
    return finish_launch(what);
}
}  // namespace

extern "C" {

size_t cfh_fused_core_workspace_bytes(const cfh_params* p, int64_t N, int64_t E, int64_t B, int32_t backward) {
    if (check_core_params(p) != CFH_OK) return 0;
    return core_layout(p, N, E, B, backward != 0).total;
}

int32_t cfh_fused_core_hist_words(const cfh_params* p) {
    if (check_core_params(p) != CFH_OK) return 0;
    return cfh::core_hist_words(p->angle_bins);
}

int cfh_fused_core_forward(const cfh_params* p, const float* qs, const float* k, const float* v, const float* a_ih,
                           const float* rpos, const float* tvecs, const float* rvlen, const int64_t* batch,
                           const int64_t* edges, const int64_t* e_start, const int32_t* order, const float* W_dist,
                           const float* W_axis1, const float* W_axis2, const float* W_axis3, int64_t N, int64_t E,
                           int64_t B, float* frames, int32_t search_frames, float* z, float* prob, float* hist,
                           float* out, const cfh_core_cache* cache, void* workspace, size_t workspace_bytes,
                           void* stream) {
    int rc = check_core_params(p);
    if (rc) return rc;
    if ((rc = check_geometry(a_ih, rpos, tvecs, batch, edges, e_start, N, E, B))) return rc;
    if ((rc = check_core_sizes(p, N, E))) return rc;
    if (N == 0) return CFH_OK;
    const bool has_ang = p->angle_bins > 0;
    if (!qs || !k || !v || !W_dist || !z || !prob || !hist || !out)
        return fail(CFH_EINVAL, "qs, k, v, W_dist, z, prob, hist and out must not be NULL");
    if (has_ang && (!W_axis1 || !W_axis2 || !W_axis3 || !frames))
        return fail(CFH_EINVAL, "the angle encoding needs W_axis1..3 and frames");
    const CoreLayout L = core_layout(p, N, E, B, false);
    if ((rc = check_workspace(workspace, workspace_bytes, L.total))) return rc;
    hipStream_t st = (hipStream_t)stream;
    char* ws = reinterpret_cast<char*>(workspace);
    cfh::CoreArgs C;
    std::memset(&C, 0, sizeof(C));
    fill_common(C.K, p, a_ih, rpos, tvecs, rvlen, batch, edges, e_start, order, N, E, workspace);
    C.K.contiguous_neighbours = 1;
    const CoreBuffers buf = fill_core(C, p, L, qs, k, v, rvlen != nullptr, cache, workspace);
    const bool search = has_ang && search_frames != 0;
    if (buf.table && !buf.table_ready) {
        TimedScope timed("core_tables", st);
        hipLaunchKernelGGL(cfh::sorted_shifts_kernel, dim3((unsigned)B), dim3(cfh::FC_TCAP), 0, st, tvecs, C.table_R,
                           buf.table);
        if (buf.near && E > 0) {
            const int s0 = 2 * C.table_R + 1;
            hipLaunchKernelGGL(cfh::pair_nearest_kernel, dim3((unsigned)((E * 8 + 255) / 256)), dim3(256), 0, st, rpos, edges,
                               batch, buf.table, s0 * s0 * s0, (int)E, buf.near);
        }
    }
    C.pair_near = buf.near;
    float* wcat = buf.wcat;
    const cfh::WcatArgs WA{W_dist, W_axis1, W_axis2, W_axis3, L.hw, p->dist_coef, p->angle_coef, p->angle_wscale, wcat};
    {
        const int prep_blocks = L.prep_blocks;
        // records whose box is not the table's are listed by the launch that makes them and taken first by the main kernel
        if (buf.table) {
            C.K.slow_count = reinterpret_cast<int32_t*>(ws + L.slow);
            C.K.slow_list = C.K.slow_count + prep_blocks;
            C.K.slow_R = C.table_R;
        }
        // the item records and the concatenated weights in one launch
        if (search) {
            // records with the query, frame search through the first set of queues; it leaves the frames in the
            // records and the main kernel takes the second set of queues
            cfh::CoreArgs F = C;
            F.K.q = qs; F.K.k = k; F.K.out_frame = frames;
            F.K.counters2 = reinterpret_cast<int32_t*>(ws + QUEUE_OFFSET + QUEUE_SET_BYTES);
            F.K.frames_to_records = 1;
            {
                TimedScope timed("core_prepare", st);
                hipLaunchKernelGGL(cfh::core_prepare_wcat_kernel, dim3(prep_blocks + p->num_heads * cfh::DH), dim3(256), 0, st,
                                   F.K, 1, prep_blocks, WA);
            }
            if (F.sorted_tab) {
                // four heads of an atom per wavefront for the items with the usual box and short rows, the others one
                // by one, all in one launch
                const unsigned item_blocks = ((unsigned)N * (unsigned)p->num_heads + cfh::CORE_WPB - 1) / cfh::CORE_WPB;
                const unsigned quad_waves = (unsigned)N * (unsigned)((p->num_heads + cfh::FQ_ROWS - 1) / cfh::FQ_ROWS);
                const unsigned quad_blocks = (quad_waves + cfh::CORE_WPB - 1) / cfh::CORE_WPB;
                if (F.K.slow_count) {
                    F.slow_lists = prep_blocks;
                    F.slow_stride = cfh::SLOW_PREP_SLOTS;
                    F.slow_wgs = slow_wave_count(N, p->num_heads);
                }
                const unsigned slow_blocks = ((unsigned)F.slow_wgs + cfh::CORE_WPB - 1) / cfh::CORE_WPB;
                {
                    TimedScope timed("frame_axes", st);
                    hipLaunchKernelGGL(cfh::frame_axes_kernel, dim3(slow_blocks + quad_blocks + item_blocks),
                                       dim3(cfh::WAVE * cfh::CORE_WPB), 0, st, F, (int)slow_blocks, (int)quad_blocks);
                }
                if ((rc = finish_launch("frame_axes"))) return rc;
            } else if ((rc = launch_core(cfh::frame_axes_sorted_kernel, F, st, "frame_axes"))) return rc;
            C.K.counters = F.K.counters2;
        } else {
            C.K.frames = has_ang ? frames : nullptr;
            TimedScope timed("core_prepare", st);
            hipLaunchKernelGGL(cfh::core_prepare_wcat_kernel, dim3(prep_blocks + p->num_heads * cfh::DH), dim3(256), 0, st,
                               C.K, 0, prep_blocks, WA);
        }
    }
    C.out = out; C.prob = prob; C.z = z; C.hist = hist;
    if (C.K.slow_count) {
        C.slow_lists = L.prep_blocks;
        C.slow_stride = cfh::SLOW_PREP_SLOTS;
        C.slow_wgs = slow_wave_count(N, p->num_heads);
    }
    C.slow_flag = cfh::REC_BOX_LISTED;
    const bool wide = p->window_mode == CFH_WINDOW_WIDE;
    const bool dyn = dist_window_dynamic(p);      // a distance window whose width is not one of the compiled ones
    const char* what = "fused_core_forward";
#define CFH_CORE_DISPATCH(KERNEL)                                                                         \
    do {                                                                                                  \
        if (p->angle_bins == cfh::SMALL_A) {                                                              \
            if (wide) rc = p->cos_abs ? (dyn ? launch_core(KERNEL<0, cfh::SMALL_A, true>, C, st, what) : launch_core(KERNEL<11, cfh::SMALL_A, true>, C, st, what))          \
                                      : (dyn ? launch_core(KERNEL<0, cfh::SMALL_A, false>, C, st, what) : launch_core(KERNEL<11, cfh::SMALL_A, false>, C, st, what));        \
            else rc = p->cos_abs ? (dyn ? launch_core(KERNEL<0, cfh::SMALL_A, true>, C, st, what) : launch_core(KERNEL<9, cfh::SMALL_A, true>, C, st, what))                \
                                 : (dyn ? launch_core(KERNEL<0, cfh::SMALL_A, false>, C, st, what) : launch_core(KERNEL<9, cfh::SMALL_A, false>, C, st, what));              \
        } else if (has_ang) {                                                                             \
            if (wide) rc = p->cos_abs ? (dyn ? launch_core(KERNEL<0, cfh::NBINS, true>, C, st, what) : launch_core(KERNEL<11, cfh::NBINS, true>, C, st, what))            \
                                      : (dyn ? launch_core(KERNEL<0, cfh::NBINS, false>, C, st, what) : launch_core(KERNEL<11, cfh::NBINS, false>, C, st, what));          \
            else rc = p->cos_abs ? (dyn ? launch_core(KERNEL<0, cfh::NBINS, true>, C, st, what) : launch_core(KERNEL<9, cfh::NBINS, true>, C, st, what))                  \
                                 : (dyn ? launch_core(KERNEL<0, cfh::NBINS, false>, C, st, what) : launch_core(KERNEL<9, cfh::NBINS, false>, C, st, what));                \
        } else {                                                                                          \
            rc = wide ? (dyn ? launch_core(KERNEL<0, 0, false>, C, st, what) : launch_core(KERNEL<11, 0, false>, C, st, what))                                    \
                      : (dyn ? launch_core(KERNEL<0, 0, false>, C, st, what) : launch_core(KERNEL<9, 0, false>, C, st, what));                                    \
        }                                                                                                 \
    } while (0)
    CFH_CORE_DISPATCH(cfh::fused_core_fwd_kernel);
    if (rc) return rc;
    {
        TimedScope timed("core_project", st);
        hipLaunchKernelGGL(cfh::core_project_kernel, dim3((unsigned)((N + 15) / 16), p->num_heads),
                           dim3(cfh::WAVE * cfh::PROJ_WAVES), 0, st, hist, wcat, out, (int)N, p->num_heads, L.hw);
    }
    return finish_launch("fused_core_project");
}

int cfh_fused_core_backward(const cfh_params* p, const float* qs, const float* k, const float* v, const float* a_ih,
                            const float* rpos, const float* tvecs, const float* rvlen, const int64_t* batch,
                            const int64_t* edges, const int64_t* e_start, const int32_t* order, const float* W_dist,
                            const float* W_axis1, const float* W_axis2, const float* W_axis3, const float* frames,
                            const float* z, const float* prob, const float* hist, const float* out, const float* gout,
                            int64_t N, int64_t E, int64_t B, float* gq, float* gk, float* gv, float* ga, float* glogit,
                            float* gW_dist, float* gW_axis1, float* gW_axis2, float* gW_axis3,
                            const cfh_core_cache* cache, void* workspace, size_t workspace_bytes, void* stream) {
    int rc = check_core_params(p);
    if (rc) return rc;
    if ((rc = check_geometry(a_ih, rpos, tvecs, batch, edges, e_start, N, E, B))) return rc;
    if ((rc = check_core_sizes(p, N, E))) return rc;
    hipStream_t st = (hipStream_t)stream;
    const bool has_ang = p->angle_bins > 0;
    const int per_enc = p->num_heads * cfh::DH * cfh::NBINS;
    if (N == 0) {
        const int per_axis = p->num_heads * cfh::DH * p->angle_bins;      // (the axes' rows have angle_bins words)
        hipLaunchKernelGGL(cfh::zero_outputs_kernel, dim3((per_enc + 255) / 256), dim3(256), 0, st, per_enc, gW_dist,
                           (float*)nullptr, (float*)nullptr, (float*)nullptr);
        if (per_axis > 0)
            hipLaunchKernelGGL(cfh::zero_outputs_kernel, dim3((per_axis + 255) / 256), dim3(256), 0, st, per_axis,
                               (float*)nullptr, gW_axis1, gW_axis2, gW_axis3);
        return finish_launch("zero_outputs");
    }
    if (!qs || !k || !v || !W_dist || !z || !prob || !hist || !out || !gout || !gq || !gk || !gv || !ga || !glogit)
        return fail(CFH_EINVAL, "fused core backward: a required pointer is NULL");
    if (has_ang && (!W_axis1 || !W_axis2 || !W_axis3 || !frames))
        return fail(CFH_EINVAL, "the angle encoding needs W_axis1..3 and frames");
    const CoreLayout L = core_layout(p, N, E, B, true);
    if ((rc = check_workspace(workspace, workspace_bytes, L.total))) return rc;
    char* ws = reinterpret_cast<char*>(workspace);
    float* gwcat = reinterpret_cast<float*>(ws + L.gwcat);
    float* G = reinterpret_cast<float*>(ws + L.G);
    cfh::CoreArgs C;
    std::memset(&C, 0, sizeof(C));
    fill_common(C.K, p, a_ih, rpos, tvecs, rvlen, batch, edges, e_start, order, N, E, workspace);
    C.K.contiguous_neighbours = 1;
    const CoreBuffers buf = fill_core(C, p, L, qs, k, v, rvlen != nullptr, cache, workspace);
    float* wcat = buf.wcat;
    C.K.frames = has_ang ? frames : nullptr;
    C.K.out_ga = ga;
    C.z = const_cast<float*>(z); C.prob = const_cast<float*>(prob);
    C.go = gout; C.outv = out; C.G = G; C.gq = gq; C.glogit = glogit;

    // ---- weight gradients: gwcat = sum_i go_i (x) hist_i, then back through the moment matrices.  They read
    //      nothing that this call makes, so they go to the second stream, beside the kernels below.
    const bool no_wg = (p->flags & CFH_FLAG_NO_WEIGHT_GRADS) != 0;      // the caller makes them later, for several calls at once
    const bool two = !(p->flags & CFH_FLAG_SINGLE_STREAM) && !no_wg;
    std::unique_lock<std::mutex> side_lock(g_side_mutex, std::defer_lock);
    SideStream* side = nullptr;
    hipStream_t st_w = st;
    if (two) {
        side_lock.lock();
        side = side_stream();
        if (!side) return fail(CFH_ELAUNCH, "second stream for the weight gradients could not be created");
        if (hipEventRecord(side->fork, st) != hipSuccess || hipStreamWaitEvent(side->stream, side->fork, 0) != hipSuccess)
            return fail(CFH_ELAUNCH, "fork to the second stream failed: %s", hipGetErrorString(hipGetLastError()));
        st_w = side->stream;
    }
    auto weight_gradients = [&]() {
        int cus = device_cus();
        if (cus <= 0) cus = 256;
        const int blocks_per_slice = (L.hw / 64) * p->num_heads;
        int nslices = (cus * 4 + blocks_per_slice - 1) / blocks_per_slice;      // about one wavefront per SIMD
        if (nslices < 1) nslices = 1;
        if (nslices > cfh::CORE_GW_SLICES) nslices = cfh::CORE_GW_SLICES;
        int per_slice = (int)((N + nslices - 1) / nslices);
        per_slice = (per_slice + 15) & ~15;
        nslices = (int)((N + per_slice - 1) / per_slice);
        TimedScope timed("core_weight_gradients", st_w);
        hipLaunchKernelGGL(cfh::core_gwcat_kernel, dim3((L.hw / 64 + cfh::GW_WPB - 1) / cfh::GW_WPB, p->num_heads, nslices),
                           dim3(cfh::WAVE * cfh::GW_WPB), 0, st_w, gout,
                           hist, gwcat, (int)N, p->num_heads, L.hw, per_slice);
        hipLaunchKernelGGL(cfh::core_gw_finish_kernel, dim3(p->num_heads * cfh::DH), dim3(256), 0, st_w, gwcat, nslices,
                           p->num_heads, L.hw, p->dist_coef, p->angle_coef, p->angle_wscale, gW_dist, gW_axis1, gW_axis2,
                           gW_axis3);
        return finish_launch("fused_core_weight_gradients");
    };
    int rc_w = CFH_OK;
    if (two) rc_w = weight_gradients();

    // ---- this stream: Wcat, G = Wcat^T go per item, records, tables, the main kernel, gk and gv
    if (!buf.wcat_ready) {
        TimedScope timed("core_prepare_bwd", st);
        hipLaunchKernelGGL(cfh::core_wcat_kernel, dim3(p->num_heads * cfh::DH), dim3(256), 0, st,
                           cfh::WcatArgs{W_dist, W_axis1, W_axis2, W_axis3, L.hw, p->dist_coef, p->angle_coef,
                                         p->angle_wscale, wcat});
    }
    // (with records kept from the forward the work queues are all that is left to prepare: gbuild clears them)
    // with the records kept from the forward pass, the same launch lists those that the main kernel is to take first
    cfh::SlowListArgs SL{};
    if (buf.records_ready && buf.table) {
        const int nlists = (int)(((N + 15) / 16 + cfh::SLOW_GB_BLOCKS - 1) / cfh::SLOW_GB_BLOCKS);
        SL.items = C.K.items;
        SL.count = reinterpret_cast<int32_t*>(reinterpret_cast<char*>(workspace) + L.slow);
        SL.list = SL.count + nlists;
        SL.R = C.table_R;
        C.K.slow_count = SL.count;
        C.K.slow_list = SL.list;
        C.slow_lists = nlists;
        C.slow_stride = cfh::SLOW_GB_BLOCKS * 16 * p->num_heads;
        C.slow_wgs = slow_wave_count(N, p->num_heads);
        C.slow_flag = cfh::REC_BOX_LISTED_BWD;
    }
    {
        TimedScope timed("core_gbuild", st);
        hipLaunchKernelGGL(cfh::core_gbuild_kernel, dim3((unsigned)((N + 15) / 16), p->num_heads, L.hw / 64), dim3(cfh::WAVE), 0,
                           st, gout, wcat, G, (int)N, p->num_heads, L.hw, buf.records_ready ? C.K.counters : nullptr, SL);
    }
    if (!buf.records_ready) {
        TimedScope timed("core_prepare_bwd", st);
        const int threads = (int)(N * p->num_heads > (int64_t)p->num_heads * cfh::NQUEUE ? N * p->num_heads
                                                                                          : p->num_heads * cfh::NQUEUE);
        hipLaunchKernelGGL(cfh::prepare_items_kernel, dim3((threads + 255) / 256), dim3(256), 0, st, C.K, 0);
    }
    if (buf.table && !buf.table_ready)
        hipLaunchKernelGGL(cfh::sorted_shifts_kernel, dim3((unsigned)B), dim3(cfh::FC_TCAP), 0, st, tvecs, C.table_R,
                           buf.table);
    const bool wide = p->window_mode == CFH_WINDOW_WIDE;
    const bool dyn = dist_window_dynamic(p);      // a distance window whose width is not one of the compiled ones
    const char* what = "fused_core_backward";
    CFH_CORE_DISPATCH(cfh::fused_core_bwd_kernel);
#undef CFH_CORE_DISPATCH
    if (!rc) {
        // gk, gv: sums over the pairs that point at an atom
        cfh::DpaArgs A;
        std::memset(&A, 0, sizeof(A));
        A.q = qs; A.k = k; A.v = v; A.edges = edges; A.e_start = e_start;
        A.prob = const_cast<float*>(prob); A.go = gout; A.gk = gk; A.gv = gv; A.gaij = glogit;
        A.N = (int32_t)N; A.H = p->num_heads; A.E = (int32_t)E;
        A.items = C.K.items;
        const int64_t items = N * p->num_heads;
        {
            TimedScope timed("core_bwd_col", st);
            hipLaunchKernelGGL(cfh::dpa_bwd_col_kernel, dim3((unsigned)((items + cfh::DPA_WAVES - 1) / cfh::DPA_WAVES)),
                               dim3(cfh::WAVE * cfh::DPA_WAVES), 0, st, A);
        }
        rc = finish_launch("fused_core_backward");
    }
    if (!two && !no_wg) rc_w = weight_gradients();
    // the join is enqueued whatever happened in between: a stream that was pulled into a capture must come back
    if (two && !(p->flags & CFH_FLAG_DEFER_JOIN) &&
        (hipEventRecord(side->join, side->stream) != hipSuccess || hipStreamWaitEvent(st, side->join, 0) != hipSuccess) &&
        !rc && !rc_w)
        rc_w = fail(CFH_ELAUNCH, "join of the second stream failed");
    return rc ? rc : rc_w;
}


size_t cfh_fused_core_weight_gradients_workspace_bytes(const cfh_params* p, int32_t njobs) {
    if (check_core_params(p) != CFH_OK || njobs < 0) return 0;
    const size_t hw = (size_t)cfh::core_hist_words(p->angle_bins);
    // (behind the header of every workspace of the library: status word, statistics, work queues)
    return COUNTER_BYTES +
           align256((size_t)cfh::CORE_GW_SLICES * p->num_heads * cfh::DH * hw * sizeof(float)) * (size_t)(njobs > 0 ? njobs : 1);
}

int cfh_fused_core_weight_gradients(const cfh_params* p, const cfh_core_wgrad_job* jobs, int32_t njobs,
                                    void* workspace, size_t workspace_bytes, void* stream) {
    int rc = check_core_params(p);
    if (rc) return rc;
    if (njobs < 0 || (njobs > 0 && !jobs)) return fail(CFH_EINVAL, "jobs is NULL or njobs negative");
    if (njobs == 0) return CFH_OK;
    const int hw = cfh::core_hist_words(p->angle_bins);
    const size_t per_job = align256((size_t)cfh::CORE_GW_SLICES * p->num_heads * cfh::DH * hw * sizeof(float));
    if ((rc = check_workspace(workspace, workspace_bytes, COUNTER_BYTES + per_job * (size_t)njobs))) return rc;
    for (int32_t j = 0; j < njobs; j++) {
        if (jobs[j].N < 0 || jobs[j].N > 0x7fffffffLL / 64)
            return fail(CFH_EINVAL, "weight-gradient job %d: N = %lld out of range", (int)j, (long long)jobs[j].N);
        if (jobs[j].N > 0 && (!jobs[j].gout || !jobs[j].hist))
            return fail(CFH_EINVAL, "weight-gradient job %d: gout and hist must not be NULL", (int)j);
    }
    hipStream_t st = (hipStream_t)stream;
    char* ws = reinterpret_cast<char*>(workspace) + COUNTER_BYTES;
    int cus = device_cus();
    if (cus <= 0) cus = 256;
    const int blocks_per_slice = (hw / 64) * p->num_heads;
    TimedScope timed("core_weight_gradients", st);
    for (int32_t first = 0; first < njobs; first += cfh::CORE_WG_MAX_JOBS) {
        const int32_t last = njobs < first + cfh::CORE_WG_MAX_JOBS ? njobs : first + cfh::CORE_WG_MAX_JOBS;
        cfh::CoreWgradJobs T{};
        T.H = p->num_heads; T.hw = hw;
        T.dist_coef = p->dist_coef; T.angle_coef = p->angle_coef; T.ws = p->angle_wscale;
        int slices = 0;
        for (int32_t j = first; j < last; j++) {
            cfh::CoreWgradJob& J = T.job[T.njobs++];
            J.go = jobs[j].gout; J.hist = jobs[j].hist;
            J.gwcat = reinterpret_cast<float*>(ws + per_job * (size_t)j);
            J.gW[0] = jobs[j].gW_dist; J.gW[1] = jobs[j].gW_axis1; J.gW[2] = jobs[j].gW_axis2; J.gW[3] = jobs[j].gW_axis3;
            J.N = (int)jobs[j].N;
            // about two wavefronts per SIMD over all jobs of the launch
            int nslices = (cus * 8 / (last - first) + blocks_per_slice - 1) / blocks_per_slice;
            if (nslices < 1) nslices = 1;
            if (nslices > cfh::CORE_GW_SLICES) nslices = cfh::CORE_GW_SLICES;
            int per_slice = (int)((jobs[j].N + nslices - 1) / nslices);
            per_slice = (per_slice + 15) & ~15;
            if (per_slice < 16) per_slice = 16;
            nslices = (int)((jobs[j].N + per_slice - 1) / per_slice);
            if (nslices < 1) nslices = 1;      // (no atoms: one slice of zeros)
            J.per_slice = per_slice;
            J.slice0 = slices;
            J.nslices = nslices;
            slices += nslices;
        }
        if (slices > 0)
            hipLaunchKernelGGL(cfh::core_gwcat_multi_kernel, dim3((hw / 64 + cfh::GW_WPB - 1) / cfh::GW_WPB, p->num_heads, slices),
                               dim3(cfh::WAVE * cfh::GW_WPB), 0, st, T);
        hipLaunchKernelGGL(cfh::core_gw_finish_multi_kernel, dim3(p->num_heads * cfh::DH, T.njobs), dim3(256), 0, st, T);
    }
    return finish_launch("fused_core_weight_gradients");
}

}  // extern "C"




