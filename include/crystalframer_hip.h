/*
 * crystalframer_hip.h -- C ABI of the MI355X (gfx950) kernels for CrystalFramer's periodic
 * infinitely-connected attention: real-space lattice sums, Gaussian distance value encoding,
 * dynamic max-frame selection and frame-projected angle value encoding, forward and backward.
 *
 * Every entry point takes plain device pointers and sizes, enqueues its kernels on the HIP stream
 * it is given (NULL = the default stream) and returns without synchronising.  The return value is
 * 0 on success or a negative CFH_E* code; cfh_last_error() then describes the failure.  The library
 * allocates nothing: scratch memory comes in through the `workspace` argument, whose required
 * size cfh_workspace_bytes() reports.  All floating-point tensors are contiguous float32, all
 * index tensors contiguous int64, exactly as the reference passes them to its kernels.
 *
 * Tensor naming (N atoms, E ordered atom pairs, B crystals, H heads, Dh head dim, K distance bins,
 * A angle bins):
 *   a_ih    (N,H)      Gaussian coefficient, a < 0            rpos   (E,3)   pos[j]-pos[i]
 *   tvecs   (B,3,3)    lattice vectors as rows                 rvlen  (B,3)   |reciprocal rows|
 *   batch   (N)        crystal of each atom                    edges  (2,E)   (i,j); edges of one
 *   e_start (N+1)      first edge of each atom                                 atom are contiguous
 *   order   (N) int32  optional visiting order of atoms for the work queue (NULL = natural)
 */
#ifndef CRYSTALFRAMER_HIP_H
#define CRYSTALFRAMER_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define CFH_ABI_VERSION 13

enum {
    CFH_OK = 0,
    CFH_EINVAL = -1,       /* bad argument (null pointer, unsupported constant, size mismatch) */
    CFH_EWORKSPACE = -2,   /* workspace missing or too small                                    */
    CFH_ELAUNCH = -3,      /* HIP reported an error when launching                              */
    CFH_EDEVICE = -4       /* no usable gfx950 device                                           */
};

/* Which truncation of the Gaussian bases the kernels use. */
enum {
    CFH_WINDOW_REFERENCE = 0,  /* +-4 sigma: ceil(8*wscale+1) bins, the reference kernels' rule
                                  (models/cuda_funcs/kernel_manager.py:146-147)                 */
    CFH_WINDOW_WIDE = 1        /* +-5 sigma: ceil(10*wscale+1) bins; dropped tail < 4e-6 of the peak */
};

/*
 * Scalar parameters.  They are the values the reference bakes into its kernels by text
 * substitution before NVRTC (models/cuda_funcs/kernel_manager.py:116-159) plus the scalar
 * arguments of its launches (models/cuda_funcs/real_space_framed_proj.py:66-104).
 */
typedef struct cfh_params {
    int32_t struct_size;     /* = sizeof(cfh_params), ABI check                                   */
    int32_t num_heads;       /* H      (HEAD_NUM)                                                 */
    int32_t head_dim;        /* Dh     (V_HEAD_DIM = K_HEAD_DIM); 16 is compiled                  */
    int32_t dist_bins;       /* K      (VPE_DIM); 0 or 64                                         */
    int32_t angle_bins;      /* A      (ANGLE_ENC_DIM); 0 or 64                                   */
    int32_t cos_abs;         /* COS_ABS 0/1                                                       */
    int32_t lattice_range;   /* LATTICE_RANGE: box half-width when cutoff_radius == 0             */
    int32_t minimum_range;   /* MINIMUM_RANGE: lower bound of the adaptive half-width (0 = none)  */
    int32_t window_mode;     /* CFH_WINDOW_*                                                      */
    float dist_max;          /* angstrom; bin centres (k+1)*dist_max/K                            */
    float dist_wscale;       /* sigma_dist = dist_wscale*dist_max/K                               */
    float angle_wscale;      /* sigma_angle = (cos_abs?1:2)*angle_wscale/(A-1)                    */
    float dist_coef;         /* length_rbf_mul                                                    */
    float angle_coef;        /* angle_rbf_mul                                                     */
    float cutoff_radius;     /* <0: -cutoff_radius sigmas of each head's Gaussian; 0: fixed box;
                                >0: absolute radius in angstrom                                   */
    float prune_log2;        /* translations whose weight is below 2^-prune_log2 of the largest
                                one of their pair are skipped; <= 0 evaluates every translation   */
    float symm_break_noise;  /* amplitude of the tie-breaking noise of the frame search (0 = the
                                deterministic first-wins rule)                                    */
    uint64_t noise_seed;     /* seed of that noise                                                */
    int32_t grad_coef_quirk; /* 1: backward scales like the reference (d/dz part by dist_coef,
                                dW_dist unscaled; real_space_framed_proj.py:183-184); 0: exact    */
    int32_t collect_stats;   /* 1: add term counts to the 32 uint64 totals at workspace+256 (the caller
                                zeroes them; launches never do): [0] forward translations evaluated,
                                [1] forward translations in the boxes, [2],[3] same for backward,
                                [4],[5] translations scanned by the two frame searches, [6],[7] (pair,
                                head) items of forward / backward                                   */
    uint64_t* noise_seed_dev; /* optional device word mixed into noise_seed when a frame search
                                starts: a caller that replays a captured graph advances it between
                                replays to draw fresh noise; NULL: noise_seed alone              */
    int32_t noise_seed_advance; /* 1: every frame search adds one to *noise_seed_dev after reading it
                                (in its own launch, so a replayed graph needs no extra kernel)   */
    int32_t flags;           /* CFH_FLAG_* bits                                                   */
} cfh_params;

/* cfh_params.flags: with the histograms kept by the forward, cfh_framed_pe_backward sums the weight
 * gradients in a kernel of its own on a second stream of the library (forked from and joined to the
 * stream of the call by events, so the call stays ordered and capturable; the first such call on a
 * device creates the stream, under capture too).  This bit keeps everything in one kernel on the stream
 * of the call instead. */
#define CFH_FLAG_SINGLE_STREAM 1
/* cfh_framed_pe_backward leaves its second stream unjoined when it returns (only where it uses that stream):
 * the caller adds work of its own behind the library's (cfh_second_stream_get; work whose inputs were
 * complete on `stream` before the call) and then MUST call cfh_second_stream_join(stream); until then the
 * weight gradients of the call are not ordered on `stream`. */
#define CFH_FLAG_DEFER_JOIN 2
/* cfh_fused_core_backward leaves the four weight gradients out (their pointers may be NULL): the caller collects
 * (gout, hist) of its calls and makes them together with cfh_fused_core_weight_gradients, e.g. for all layers when a
 * backward pass ends, away from the main kernels that they would otherwise run beside. */
#define CFH_FLAG_NO_WEIGHT_GRADS 4

/*
 * The library's second stream of the current device, for a caller that has work of its own to run beside
 * the gather-only kernel of cfh_framed_pe_backward (the Python mirror sends the weight gradients of the
 * linear layers collected so far).  cfh_second_stream_fork makes that stream wait for everything enqueued
 * on `stream` so far and returns it in *second; what the caller enqueues there must be joined before
 * `stream` (or the host) relies on it, by cfh_second_stream_join(stream).  Memory the enqueued work touches
 * must stay allocated until then.  One thread per device at a time.  No counterpart in the reference.
 */
int cfh_second_stream_fork(void* stream, void** second);
/* The same stream without making it wait: for work that may run as soon as what is already on it is done. */
int cfh_second_stream_get(void** second);
int cfh_second_stream_join(void* stream);

/* Version of this ABI; a mismatch with CFH_ABI_VERSION means header and library differ. */
int cfh_abi_version(void);

/* Text of the last error on the calling thread ("" if none). */
const char* cfh_last_error(void);

/*
 * Diagnostics with no counterpart in the reference.  After cfh_timing_enable(1) every call of the
 * frame-search and value-encoding entry points brackets its lattice-sum kernel (that kernel alone,
 * not the small kernels around it) with HIP events on the stream of the call; cfh_timing_read waits
 * for the launches recorded under `what` ("frame_axis1", "frame_axis2", "frame_axes",
 * "framed_pe_forward", "framed_pe_backward"), returns their summed duration and count, and forgets
 * them.  Not to be enabled while the stream is being captured into a graph.
 */
int cfh_timing_enable(int on);
int cfh_timing_read(const char* what, double* total_ms, int64_t* launches);

/* Bytes of device scratch the four entry points below need for (N atoms, E pairs).  The first 512 bytes of
 * a workspace are a header that the caller zeroes once: bytes 0..7 the snapshot of the noise seed, the int32
 * at byte 16 a status word of flag bits that launches set and never clear: 1 when the box rule asked for a
 * half-width beyond 32 (the largest the kernels sum; the box was cut back and the result differs from the
 * reference's), 2 when a call of the fused core found pairs that are not the complete n x n block of every crystal
 * sorted by i then j (every read stays inside the arrays, the results are meaningless); bytes 256..511 the
 * statistics of collect_stats. */
size_t cfh_workspace_bytes(const cfh_params* p, int64_t N, int64_t E);

/*
 * First frame axis, f1 (N,H,3): unit vector towards the nearest periodic image (d^2 > 1e-5) of the
 * neighbour j maximising  q_i.k_j + a_ih*d2min(i,j).  `q` (N,H,Dh) must already be divided by
 * sqrt(Dh); `k` (N,H,Dh).
 * Replaces ComputeFrame1MaximumMethodCUDA.forward: kernel compute_maximum_frame_each_edge, the
 * gathered q.k product and torch_scatter.scatter_max
 * (models/cuda_funcs/calc_maximum_frame.py:24-87, models/kernels/compute_maximum_frame_each_edge.cu).
 */
int cfh_frame_axis1(const cfh_params* p, const float* q, const float* k, const float* a_ih,
                    const float* rpos, const float* tvecs, const float* rvlen,
                    const int64_t* batch, const int64_t* edges, const int64_t* e_start,
                    const int32_t* order, int64_t N, int64_t E, int64_t B,
                    float* frame1, void* workspace, size_t workspace_bytes, void* stream);

/*
 * Second frame axis before orthogonalisation, f2max (N,H,3): unit vector towards the image (over
 * all neighbours j and translations n) maximising
 *   q_i.k_j + a_ih*d^2 + log(max(1-|cos(image, f1)|, 1e-5)),   |cos| < 0.9999, d^2 > 1e-5.
 * Replaces ComputeFrame2MaximumMethodCUDA.forward
 * (models/cuda_funcs/calc_maximum_frame.py:95-166, models/kernels/compute_second_frame_each_edge.cu).
 */
int cfh_frame_axis2(const cfh_params* p, const float* q, const float* k, const float* a_ih,
                    const float* rpos, const float* tvecs, const float* rvlen,
                    const int64_t* batch, const int64_t* edges, const int64_t* e_start,
                    const int32_t* order, const float* frame1, int64_t N, int64_t E, int64_t B,
                    float* frame2max, void* workspace, size_t workspace_bytes, void* stream);

/*
 * Both searches above in one launch, followed by the orthogonalisation the reference does in PyTorch:
 * frames (3,N,H,3) = (f1, normalize(f2max - (f1.f2max) f1), f1 x f2).
 * Replaces compute_frame_maximum_method_ for frame_method "max"
 * (models/indexed_lattice_multi_head_attention_cuda.py:455-481).
 */
int cfh_frame_axes(const cfh_params* p, const float* q, const float* k, const float* a_ih,
                   const float* rpos, const float* tvecs, const float* rvlen, const int64_t* batch,
                   const int64_t* edges, const int64_t* e_start, const int32_t* order, int64_t N,
                   int64_t E, int64_t B, float* frames, void* workspace, size_t workspace_bytes,
                   void* stream);

/*
 * z (E,H) = log sum_n exp(a_ih*|rpos + n.L|^2) and, when K > 0, the value position encoding
 * psi (E,H,Dh) = dist_coef * W_dist.s_dist + angle_coef * sum_axis W_axis.s_axis, where s are the
 * softmax-over-translations averages of the truncated Gaussian bases of the distance and of the
 * cosine to each frame axis.  W_dist (H,Dh,K); W_axis[3] each (H,Dh,A) or all NULL; frames
 * (3,N,H,3) or NULL.  d2min_out (E,H) is optional.  shat_out (E,H,4,64) is optional: when given,
 * the softmax-averaged basis values s (the window histograms, rows: distance, axis 1..3) are kept
 * for cfh_framed_pe_backward, which then rebuilds nothing (1 KB per (pair, head) of HBM against
 * about a third of the backward's time).
 * Replaces RealEncodingWithFramedProjFuncCUDA.forward: kernels real_enc_frame_proj_fwd_length and
 * real_enc_frame_proj_fwd_angle and the sums between them
 * (models/cuda_funcs/real_space_framed_proj.py:21-120).
 */
int cfh_framed_pe_forward(const cfh_params* p, const float* a_ih, const float* rpos,
                          const float* tvecs, const float* rvlen, const int64_t* batch,
                          const int64_t* edges, const int64_t* e_start, const int32_t* order,
                          const float* W_dist, const float* W_axis1, const float* W_axis2,
                          const float* W_axis3, const float* frames, int64_t N, int64_t E,
                          int64_t B, float* z, float* psi, float* d2min_out, float* shat_out,
                          void* workspace, size_t workspace_bytes, void* stream);

/*
 * cfh_framed_pe_forward without the workspace argument: the scratch of its kernels (work-queue heads and the
 * per-(atom, head) records) is a file-scope device array of the library, CFH_STATIC_MAX_ITEMS records plus the
 * queue heads (about 8.5 MB, held by every GPU the library has run on until the process ends).  It has no
 * counterpart in the reference: it is for callers that cannot allocate device memory or hand over a workspace --
 * code under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc.  The call allocates
 * nothing.  Same arguments, results and errors as cfh_framed_pe_forward otherwise; N * num_heads beyond
 * CFH_STATIC_MAX_ITEMS and collect_stats return CFH_EINVAL.  All calls on one GPU share the one array: calls
 * that overlap on a GPU (two streams, two threads) race; calls on one stream are ordered and safe.
 */
#define CFH_STATIC_MAX_ITEMS 65536
int cfh_framed_pe_forward_static(const cfh_params* p, const float* a_ih, const float* rpos,
                                 const float* tvecs, const float* rvlen, const int64_t* batch,
                                 const int64_t* edges, const int64_t* e_start, const int32_t* order,
                                 const float* W_dist, const float* W_axis1, const float* W_axis2,
                                 const float* W_axis3, const float* frames, int64_t N, int64_t E,
                                 int64_t B, float* z, float* psi, float* d2min_out, float* shat_out,
                                 void* stream);

/*
 * cfh_frame_axes followed by cfh_framed_pe_forward with the frames it found, as the attention layer
 * calls them (models/indexed_lattice_multi_head_attention_cuda.py:666-734: compute_frame_maximum_method_,
 * then RealEncodingWithFramedProjFuncCUDA.apply): same arguments and results as the two calls (`frames`
 * (3,N,H,3) is an output here), one launch less -- the per-item records (box, lattice, coefficient) are
 * built once, the search stores its frames into them and the forward kernel works through them with a
 * second set of work queues.
 */
int cfh_frame_axes_framed_pe_forward(const cfh_params* p, const float* q, const float* k, const float* a_ih,
                                     const float* rpos, const float* tvecs, const float* rvlen,
                                     const int64_t* batch, const int64_t* edges, const int64_t* e_start,
                                     const int32_t* order, const float* W_dist, const float* W_axis1,
                                     const float* W_axis2, const float* W_axis3, int64_t N, int64_t E,
                                     int64_t B, float* frames, float* z, float* psi, float* d2min_out,
                                     float* shat_out, void* workspace, size_t workspace_bytes, void* stream);

/*
 * Gradients of the above for upstream gz (E,H) and gpsi (E,H,Dh): ga (N,H), gW_dist (H,Dh,K),
 * gW_axis[3] (H,Dh,A).  The per-translation weights are recomputed from z, not stored.  The
 * weight gradients are returned already summed over atoms.  No gradient flows to the frames
 * (the reference returns None for them).  `shat` is what the forward wrote to shat_out, or NULL
 * (the histograms are then rebuilt, as the reference does).
 * Replaces RealEncodingWithFramedProjFuncCUDA.backward: kernels real_enc_frame_proj_bwd_length and
 * real_enc_frame_proj_bwd_angle (models/cuda_funcs/real_space_framed_proj.py:123-221).
 */
int cfh_framed_pe_backward(const cfh_params* p, const float* a_ih, const float* rpos,
                           const float* tvecs, const float* rvlen, const int64_t* batch,
                           const int64_t* edges, const int64_t* e_start, const int32_t* order,
                           const float* W_dist, const float* W_axis1, const float* W_axis2,
                           const float* W_axis3, const float* frames, const float* z,
                           const float* gz, const float* gpsi, const float* shat, int64_t N,
                           int64_t E, int64_t B, float* ga, float* gW_dist, float* gW_axis1,
                           float* gW_axis2, float* gW_axis3, void* workspace, size_t workspace_bytes,
                           void* stream);

/*
 * Attention over the pairs of each atom: l_e = q_i.k_j + aij_e, p = softmax over the pairs (i,.)
 * of atom i, out_i = sum_e p_e (v_j + bij_e).  q (already divided by sqrt(Dh)), k, v, out (N,H,Dh);
 * aij (E,H) or NULL; bij (E,H,Dh) or NULL; prob (E,H) receives the attention weights (the backward
 * needs them).  Dh = 16.  Needs no workspace.
 * Replaces FusedDotProductAttentionCUDA.forward: kernel fused_dpa_fwd
 * (models/cuda_funcs/fused_dpa.py:17-63, models/kernels/fused_dpa_fwd.cu).
 */
int cfh_fused_dpa_forward(const float* q, const float* k, const float* v, const float* aij,
                          const float* bij, const int64_t* edges, const int64_t* e_start, int64_t N,
                          int64_t H, int64_t Dh, int64_t E, float* prob, float* out, void* stream);

/*
 * Gradients of the above for upstream gout (N,H,Dh): gq, gk, gv (N,H,Dh), gaij (E,H; always
 * written, also when aij was NULL) and gbij (E,H,Dh) or NULL.  The pairs must be the complete
 * n x n block of every crystal with rows and columns in atom order (cfh_pair_layout_check), which
 * is what lets gk and gv be summed without atomics and without the transposed copies the
 * reference makes.
 * Replaces FusedDotProductAttentionCUDA.backward: kernels irregular_transpose, fused_dpa_bwd and
 * fused_dpa_bwd_q (models/cuda_funcs/fused_dpa.py:65-170).
 */
int cfh_fused_dpa_backward(const float* q, const float* k, const float* v, const float* aij,
                           const float* bij, const int64_t* edges, const int64_t* e_start,
                           const float* prob, const float* out, const float* gout, int64_t N,
                           int64_t H, int64_t Dh, int64_t E, float* gq, float* gk, float* gv,
                           float* gaij, float* gbij, void* stream);

/*
 * ga (N,H) of cfh_framed_pe_backward when the projection weights differ from pair to pair (W_num = E or N in
 * models/kernels/real_enc_frame_proj_bwd_length.cu:166-173, models/cuda_funcs/real_space_framed_proj.py:156): the
 * kernel needs the weights only through the rows g = W^T gpsi, which the caller makes for every pair,
 *     g_pair[e,h,0,k] = dist_coef  sum_c W_dist[w(e),h,c,k] gpsi[e,h,c],
 *     g_pair[e,h,1+axis,k] = angle_coef sum_c W_axis[w(e),h,c,k] gpsi[e,h,c]        (E,H,4,64; unused rows and, for a
 * 16-bin angle basis, the entries beyond the bins: zero), and the weight gradients are outer products of gpsi and the
 * histograms of the forward (shat), the caller's as well.  frames NULL: no angle encoding.
 */
int cfh_framed_pe_backward_pairwise(const cfh_params* p, const float* a_ih, const float* rpos, const float* tvecs,
                                    const float* rvlen, const int64_t* batch, const int64_t* edges,
                                    const int64_t* e_start, const int32_t* order, const float* frames, const float* z,
                                    const float* gz, const float* g_pair, int64_t N, int64_t E, int64_t B, float* ga,
                                    void* workspace, size_t workspace_bytes, void* stream);

/*
 * The attention core of a layer in one call: lattice sums, softmax over the pairs of every atom and the value
 * encoding, with the "max" frame search in front when search_frames != 0 (frames (3,N,H,3) is then an output,
 * else an input; unused without the angle encoding):
 *     out_i = sum_j P_ij (v_j + psi_ij),  P_i. = softmax_j (qs_i . k_j + z_ij),
 * i.e. cfh_frame_axes, cfh_framed_pe_forward and cfh_fused_dpa_forward composed
 * (models/indexed_lattice_multi_head_attention_cuda.py:589-734 and :144-185; models/cuda_funcs/fused_dpa.py:17-63),
 * computed differently: because out is linear in psi = W . s, the basis values of all images of all pairs of an
 * atom are scattered, weighted by P_ij p_n, into ONE histogram per (atom, head), which is projected once.
 * psi (E,H,Dh) and the per-pair histograms are never formed.  The distance basis keeps the truncated window of
 * window_mode (CFH_WINDOW_WIDE, +-5 sigma: full-basis results to within 4e-6 of a basis function's peak); the angle
 * basis is the FULL Gaussian basis (no truncation: the pure-PyTorch formulation,
 * models/indexed_lattice_multi_head_attention.py:580-588): with 64 bins evaluated as a 5-term series around the
 * nearest bin (error < 2e-6 of a basis function's peak for angle_wscale 4; angle_wscale < 3 returns CFH_EINVAL), with
 * 16 bins (the reference's lightweight setting, train_jarvis_time.sh:40-57; angle_wscale >= 1) by adding all 16
 * basis values of every image, as the reference evaluates that basis.
 * Needs dist_bins = 64, dist_wscale = 1, angle_bins 0, 16 or 64, and the pairs as the complete n x n block of every
 * crystal (cfh_pair_layout_check; a call that finds another layout sets bit 2 of the workspace's status word).
 * qs = query / sqrt(Dh).
 * Results kept for the backward: z (E,H), prob (E,H) = P, hist (H,N,words) the normalised histograms
 * (head-major: the kernels that contract them with the weights read the rows of a head one after the other)
 * (words = cfh_fused_core_hist_words: 64 distance bins, then per axis and order 64 moment bins = 1024; with 16
 * angle bins 64 + 3 x 16 padded to 128), out (N,H,Dh).
 * workspace: cfh_fused_core_workspace_bytes(p, N, E, B, 0).
 *
 * cache (may be NULL, as may every pointer in it): buffers the caller keeps so that later calls need not make
 * them again.  Without them the library makes each in its workspace on every call.
 *   shift_table (B,128,4)   the shifts of the (2R+1)^3 box of every crystal sorted by length (R = minimum_range with
 *                           the adaptive cutoff, else lattice_range; used when that box has at most 128 shifts and
 *                           prune_log2 > 0).  It depends on tvecs and R only: with shift_table_ready != 0 the call
 *                           reads it (filled by an earlier call, forward or backward, with the same tvecs and
 *                           params), else it fills it.
 *   pair_near (E,2)         per pair over that box: the smallest squared distance of all images and of the images
 *                           with d^2 > 1e-5, the second with the position of its image in shift_table in its low
 *                           7 bits (an opaque buffer: the library writes and reads it; geometry alone: made once
 *                           per batch, together with shift_table and
 *                           under the same ready word; the lattice sums then skip their sweep for the nearest
 *                           image and the frame search reads shorter prefixes of the table).  Only the forward
 *                           uses it; without it the forward makes it in its workspace.
 *   wcat (H,Dh,words)       the projection weights with the moment matrices folded in; the forward writes it, the
 *                           backward reads it when wcat_ready != 0 (same weights as in the forward) or makes it.
 *   records (N,H,32)        the item records of the launch (box, lattice and frames of every (atom, head)); the
 *                           forward writes them, the backward reads them when records_ready != 0 or makes them.
 */
typedef struct cfh_core_cache {
    float* shift_table;
    float* pair_near;
    float* wcat;
    uint32_t* records;
    int32_t shift_table_ready;
    int32_t wcat_ready;
    int32_t records_ready;
    int32_t reserved0;
} cfh_core_cache;

size_t cfh_fused_core_workspace_bytes(const cfh_params* p, int64_t N, int64_t E, int64_t B, int32_t backward);
int32_t cfh_fused_core_hist_words(const cfh_params* p);
int cfh_fused_core_forward(const cfh_params* p, const float* qs, const float* k, const float* v, const float* a_ih,
                           const float* rpos, const float* tvecs, const float* rvlen, const int64_t* batch,
                           const int64_t* edges, const int64_t* e_start, const int32_t* order, const float* W_dist,
                           const float* W_axis1, const float* W_axis2, const float* W_axis3, int64_t N, int64_t E,
                           int64_t B, float* frames, int32_t search_frames, float* z, float* prob, float* hist,
                           float* out, const cfh_core_cache* cache, void* workspace, size_t workspace_bytes,
                           void* stream);

/*
 * Gradients of the above for upstream gout (N,H,Dh): gq (of qs), gk, gv (N,H,Dh), ga (N,H), the four weight
 * gradients (H,Dh,64) summed over atoms; glogit (E,H) is scratch the caller provides (the gradient of the logits).
 * No gradient flows to the frames.  What FusedDotProductAttentionCUDA.backward and
 * RealEncodingWithFramedProjFuncCUDA.backward compute together (models/cuda_funcs/fused_dpa.py:65-170,
 * real_space_framed_proj.py:123-221); the weight gradients add their atoms with float atomics.
 * The weight gradients need only gout and the histograms of the forward: they are made on the library's second
 * stream beside the main kernel (forked from and joined to `stream` inside the call) unless
 * p->flags has CFH_FLAG_SINGLE_STREAM; with CFH_FLAG_DEFER_JOIN the caller joins (cfh_second_stream_join).
 * workspace: cfh_fused_core_workspace_bytes(p, N, E, B, 1).  cache: as for the forward (read when the ready words
 * say so).
 */
int cfh_fused_core_backward(const cfh_params* p, const float* qs, const float* k, const float* v, const float* a_ih,
                            const float* rpos, const float* tvecs, const float* rvlen, const int64_t* batch,
                            const int64_t* edges, const int64_t* e_start, const int32_t* order, const float* W_dist,
                            const float* W_axis1, const float* W_axis2, const float* W_axis3, const float* frames,
                            const float* z, const float* prob, const float* hist, const float* out, const float* gout,
                            int64_t N, int64_t E, int64_t B, float* gq, float* gk, float* gv, float* ga, float* glogit,
                            float* gW_dist, float* gW_axis1, float* gW_axis2, float* gW_axis3,
                            const cfh_core_cache* cache, void* workspace, size_t workspace_bytes, void* stream);

/*
 * The weight gradients of up to 8 calls of cfh_fused_core_backward made with CFH_FLAG_NO_WEIGHT_GRADS, in one launch
 * per step (products of gout with the histograms, then the way back through the moment matrices):
 *     gW_* (H,Dh,64) += sum over the atoms of gout (x) hist   (ADDED to what the destinations hold; NULL: not wanted)
 * Every job: gout (N,H,Dh) and hist (H,N,words) of one call.  p: the params of those calls (heads, bins, coefficients).
 * workspace: cfh_fused_core_weight_gradients_workspace_bytes(p, njobs) bytes.  `jobs` is a host array; it is copied
 * into the kernel arguments.  With float atomics, like the weight gradients inside cfh_fused_core_backward.
 * No counterpart in the reference (autograd sums its per-atom weight gradients, real_space_framed_proj.py:211-219).
 */
typedef struct cfh_core_wgrad_job {
    const float* gout;
    const float* hist;
    int64_t N;
    float* gW_dist;
    float* gW_axis1;
    float* gW_axis2;
    float* gW_axis3;
} cfh_core_wgrad_job;
size_t cfh_fused_core_weight_gradients_workspace_bytes(const cfh_params* p, int32_t njobs);
int cfh_fused_core_weight_gradients(const cfh_params* p, const cfh_core_wgrad_job* jobs, int32_t njobs,
                                    void* workspace, size_t workspace_bytes, void* stream);

/*
 * Sets *flag (device memory) to 0 when edges (2,E) / e_start (N+1) hold, for every crystal, all
 * n x n pairs (i,j) sorted by i then j, to 1 otherwise.  The reference relies on the same layout
 * without checking it (models/kernels/irregular_transpose.cu).
 */
int cfh_pair_layout_check(const int64_t* edges, const int64_t* e_start, int64_t N, int64_t E,
                          int32_t* flag, void* stream);

/*
 * Per-crystal mean of per-atom rows: out (B,C) from x (N,C); atom_start (B+1) are the prefix sums
 * of the crystal sizes (atoms of a crystal are contiguous).  The backward spreads gout (B,C) back:
 * gx[i] = gout[batch[i]] / size.
 * Replaces IrregularMeanCUDA: kernels irregular_mean_fwd and the gather of its backward
 * (models/cuda_funcs/irregular_mean.py:19-70).
 */
int cfh_crystal_mean_forward(const float* x, const int64_t* atom_start, int64_t N, int64_t B,
                             int64_t C, float* out, void* stream);
int cfh_crystal_mean_backward(const float* gout, const int64_t* batch, const int64_t* atom_start,
                              int64_t N, int64_t B, int64_t C, float* gx, void* stream);

/*
 * Geometry of a batch of fully connected crystals, shared by all layers of a forward pass: the pairs
 * (i, j) of every crystal as the complete n x n block, i-major (edges (2,E) int64), pair vectors
 * rpos (E,3) = pos[j] - pos[i], reciprocal rows recip (B,3,3) = 2 pi (t_b x t_c) / V etc., their lengths
 * rvlen (B,3), the signed cell volume vcell (B), e_start (N+1) first pair of each atom, atom_start (B+1)
 * first atom of each crystal and `order` (N) int32, the atoms by descending crystal size (the order
 * in which the lattice kernels take their items).  batch (N) ascending, sizes (B) atoms per crystal,
 * E = sum of sizes^2 (known to the caller; e_start[N] holds what the device counted).  workspace:
 * (2 B + 1) * 8 bytes.  Three launches.  Replaces the framework arithmetic of
 * models/indexed_latticeformer_encoder.py:15-44 (compute_lattice_distances_for_cuda) and :175-245
 * (get_edge_index).
 */
int cfh_crystal_geometry(const float* pos, const int64_t* batch, const float* tvecs, const int64_t* sizes,
                         int64_t N, int64_t B, int64_t E, int64_t* edges, float* rpos, float* recip,
                         float* rvlen, float* vcell, int64_t* e_start, int64_t* atom_start, int32_t* order,
                         void* workspace, size_t workspace_bytes, void* stream);

/*
 * Weight and bias gradients of a projection y = x W^T + b:  dW (O,I) = dy^T x, db (O) = column sums
 * of dy (db may be NULL); x (N,I), dy (N,O), row-major.  One launch (plus a clearing kernel) sized
 * for the shapes of this model, N = atoms in the thousands and I, O in the hundreds, where the
 * general GEMM plus a separate reduction take 19 + 10 us.  The reference leaves this to
 * torch.nn.functional.linear's autograd (models/indexed_lattice_multi_head_attention_cuda.py:141,988,
 * models/indexed_latticeformer_encoder.py:606).
 */
int cfh_linear_weight_bias_grad(const float* x, const float* dy, int64_t N, int64_t I, int64_t O,
                                float* dW, float* db, void* stream);

/*
 * The same gradients for several layers in one launch, ACCUMULATED into dW and db (the caller has
 * initialised them: zeros, or gradients to add to).  Each job: x (N,I) with row stride ldx, dy (N,O)
 * with row stride ldy (so a job may take a column block of a wider dy, e.g. one of the three
 * stacked input projections), dW (O,I) contiguous, db (O) or NULL.  A job with dW == NULL adds only the
 * column sums of dy to db (x is not read, I = ldx = 1): any sum over rows that a backward pass leaves
 * for its end, e.g. the per-block partials of cfh_attention_inputs_backward.  Row strides up to 2^26 elements.  A
 * job whose O and I are multiples of 64, whose strides are multiples of 4 and whose x and dy are 16-byte aligned
 * takes a faster kernel variant (16-byte loads); the results are the same up to the order of the float sums.
 * `jobs` is a host array; it is copied into the kernel arguments, 32 jobs per launch.  Deferring the weight gradients of a whole
 * backward pass to one call replaces one launch (plus clearing) per layer -- latency-bound at these
 * sizes -- by a launch that fills the chip.  No counterpart in the reference (autograd of
 * torch.nn.functional.linear, one GEMM per layer).
 *
 * The rows of a job are split over several workgroups per 64x64 tile of dW.  With workspace == NULL they add
 * their parts with float atomics (the sums differ in the last bits from run to run).  With a workspace of at
 * least cfh_linear_weight_bias_grad_batch_workspace_bytes(jobs, njobs) bytes every workgroup stores its part
 * there and a second kernel adds the parts in the order of the row slices: the same bits on every run with the
 * same jobs on the same device.  Jobs whose dW or db overlap (a weight used twice in one pass) then go to
 * separate launches, in the jobs' order.  The workspace needs no initialisation and holds nothing between calls.
 */
typedef struct cfh_linear_grad_job {
    const float* x;
    const float* dy;
    float* dW;
    float* db;
    int64_t N, I, O, ldx, ldy;
} cfh_linear_grad_job;
size_t cfh_linear_weight_bias_grad_batch_workspace_bytes(const cfh_linear_grad_job* jobs, int32_t njobs);
int cfh_linear_weight_bias_grad_batch(const cfh_linear_grad_job* jobs, int32_t njobs, void* workspace,
                                      size_t workspace_bytes, void* stream);

/*
 * One AdamW step (decoupled weight decay, bias-corrected moments; the update rule of torch.optim.AdamW without
 * amsgrad / maximize) for several parameter tensors in one launch:
 *     p *= 1 - lr wd;  m = b1 m + (1 - b1) g;  v = b2 v + (1 - b2) g^2;
 *     p -= lr / (1 - b1^t) * m / (sqrt(v) / sqrt(1 - b2^t) + eps),   t = *step_dev + 1
 * and *step_dev (device memory: the steps taken so far, 0 before the first) is advanced by one afterwards, on the
 * stream, so that a captured call keeps counting from replay to replay.  Every tensor is contiguous float32 with n
 * elements.  `jobs` is a host array; it is copied into the kernel arguments, 80 tensors per launch.  The model of
 * the benchmark has 65 small tensors (0.95 M elements): the framework's multi-tensor kernel takes 2 launches of
 * 43 us for them, bound by its per-tensor bookkeeping.  No counterpart in the reference (torch.optim.AdamW in its
 * trainer, train.py); it is here because the measured training step contains the update.
 */
typedef struct cfh_adamw_job {
    float* param;
    const float* grad;
    float* exp_avg;
    float* exp_avg_sq;
    int64_t n;
} cfh_adamw_job;
int cfh_adamw_step_batch(const cfh_adamw_job* jobs, int32_t njobs, float lr, float beta1, float beta2, float eps,
                         float weight_decay, uint64_t* step_dev, void* stream);

/*
 * Projections with few rows (one per crystal: the head after pooling), where the general GEMM runs on
 * one or two workgroups:  y (M,N) = x (M,K) W^T + b with W (N,K) as torch.nn.Linear stores it, b (N) or
 * NULL, relu != 0: max(0, .);  dx (M,K) = dy (M,N) W.  Contiguous float32; K % 16 == 0 for the forward;
 * for dx N % 16 == 0, or N <= 64 (a plain loop: the single regression target).  Replace
 * torch.nn.functional.linear and its input gradient (models/latticeformer.py,
 * the MLP head after pooling).
 */
int cfh_small_linear_forward(const float* x, const float* W, const float* b, int64_t M, int64_t N, int64_t K,
                             int32_t relu, float* y, void* stream);
int cfh_small_linear_dx(const float* dy, const float* W, int64_t M, int64_t N, int64_t K, float* dx, void* stream);

/*
 * The projections between the attention cores of two consecutive encoder layers, which act on every atom
 * separately, in one launch (forward):
 *   x1 (N,D) = x_res + attn Wo^T + bo;  h (N,F) = relu(x1 W1^T + b1);  x2 (N,D) = x1 + h W2^T + b2;
 *   with Wqkv (3D,D): qkv (N,3D) = x2 Wqkv^T + bqkv and qs, k, v, a as cfh_attention_inputs_forward makes
 *   them from qkv (Wqkv NULL: the chain ends with x2 and the last eight outputs are not touched).
 * Weights as torch.nn.Linear stores them, biases may be NULL; D = 16 H and F multiples of 128.  Every
 * intermediate is an output because the backward pass (framework GEMMs and the entry points above) needs
 * it.  Replaces, for a layer without layer norm and dropout and with the ReLU activation, the out_proj of
 * the attention and the residual (models/indexed_lattice_multi_head_attention_cuda.py:734,
 * models/indexed_latticeformer_encoder.py:639-648), the feed-forward block (:606, :644-648) and the
 * input projection, query scaling and Gaussian coefficient of the next layer
 * (models/indexed_lattice_multi_head_attention_cuda.py:399-409, :896-940): seven launches of the framework
 * per layer in the reference's formulation.
 */
int cfh_layer_bridge_forward(const float* attn, const float* x_res, int64_t N, int32_t D, int32_t F, const float* Wo,
                             const float* bo, const float* W1, const float* b1, const float* W2, const float* b2,
                             const float* Wqkv, const float* bqkv, const float* lattice_w,
                             const float* gauss_scale_dev, float c1, float lb, float c2, float q_scale, int32_t H,
                             float* x1, float* h, float* x2, float* qkv, float* qs, float* k, float* v, float* a,
                             void* stream);

/*
 * Input gradients of the chain of cfh_layer_bridge_forward in one launch:
 *   g2 (N,D) = g_x2 + gqkv Wqkv;  gh (N,F) = (g2 W2) where h > 0, else 0;  g1 (N,D) = g2 + gh W1  (the
 *   gradient of x_res and of x1);  g_attn (N,D) = g1 Wo.
 * g_x2 may be NULL (zero).  gqkv NULL (no next layer): g2 = g_x2 and g2 is not written.  gqkv is what
 * cfh_attention_inputs_backward returns; with `ai` given instead (gqkv NULL), that backward is made here as
 * well, from the gradients of (qs, k, v, a), and gqkv is an output.  All four results are outputs because the weight gradients are
 * their products with the saved activations (cfh_linear_weight_bias_grad_batch: dWqkv = gqkv^T x2,
 * dW2 = g2^T h, dW1 = gh^T x1, dWo = g1^T attn).  D, F multiples of 128; returns CFH_EINVAL when D and F
 * need more LDS than a CU has (the caller then uses GEMMs).  Replaces the framework's autograd of the same
 * modules (eight launches per layer).
 */
typedef struct cfh_attention_inputs_grad {
    const float* qkv;              /* (N, 3D) the forward's stacked projection output */
    const float* lattice_w;        /* (D) */
    const float* gauss_scale_dev;  /* device {scale, shift} or NULL */
    const float* gqs;              /* upstream gradients of qs, k, v (N,D) and a (N,H); each may be NULL (zero) */
    const float* gk;
    const float* gv;
    const float* ga;
    float* gqkv;                   /* out (N, 3D): what cfh_attention_inputs_backward would return */
    float* gw_partial;             /* out (ceil(N/16), D): per-block sums of the lattice-weight gradient; their
                                      column sums are that gradient (a dW == NULL job of the batched launch) */
    float c1, lb, c2, q_scale;
    int32_t H;
    int32_t reserved0;
} cfh_attention_inputs_grad;
int cfh_layer_bridge_backward(const float* g_x2, const float* gqkv, const float* h, const float* Wqkv,
                              const float* W2, const float* W1, const float* Wo, int64_t N, int32_t D, int32_t F,
                              float* g2, float* gh, float* g1, float* g_attn, const cfh_attention_inputs_grad* ai,
                              void* stream);

/*
 * What lies between the stacked q/k/v projection of a layer and its kernels, one launch each way.
 * Forward: qkv (N, 3 H Dh), rows = [query | key | value];  qs = query * q_scale, k, v (N,H,Dh) contiguous,
 *   a (N,H) = ((1 - lb) elu(c1 alpha') + 1) c2  with alpha = query_h . lattice_w_h and
 *   alpha' = (alpha + gauss_scale_dev[1]) * gauss_scale_dev[0]  (alpha' = alpha when the pointer is NULL).
 * Backward: gqkv (N, 3 H Dh) = [ga da/dquery + gqs q_scale | gk | gv],  g_lattice_w (H Dh) = sum over atoms
 *   of ga da/dalpha query;  gqs, gk, gv, ga may each be NULL (zero).  gauss_scale_dev is a constant.
 *   workspace: ceil(N / (4 * (256 / (H Dh)))) * H Dh floats, left holding the per-block partial sums of
 *   g_lattice_w as a (blocks, H Dh) matrix; with g_lattice_w == NULL the launch that adds them up is left
 *   out and the caller sums the columns itself (a dW == NULL job of cfh_linear_weight_bias_grad_batch).
 * Dh = 16, 256 % (H Dh) == 0.  Replaces the framework arithmetic of
 * models/indexed_lattice_multi_head_attention_cuda.py:896-940 (gaussian coefficient: c1 = beta / (1 - lb),
 * c2 = -1/2 scale_real^-2), the query scaling of :144-185 and :455, and the chunk / cat of the
 * projection output and its gradient (:399-409).
 */
int cfh_attention_inputs_forward(const float* qkv, const float* lattice_w, const float* gauss_scale_dev,
                                 float c1, float lb, float c2, float q_scale, int64_t N, int32_t H, int32_t Dh,
                                 float* qs, float* k, float* v, float* a, void* stream);
int cfh_attention_inputs_backward(const float* qkv, const float* lattice_w, const float* gauss_scale_dev,
                                  float c1, float lb, float c2, float q_scale, const float* gqs, const float* gk,
                                  const float* gv, const float* ga, int64_t N, int32_t H, int32_t Dh,
                                  float* gqkv, float* g_lattice_w, void* workspace, size_t workspace_bytes,
                                  void* stream);

#ifdef __cplusplus
}
#endif
#endif /* CRYSTALFRAMER_HIP_H */
