"""Operator boundary: ``torch.autograd.Function`` classes with the names and positional signatures
of the reference's ``models/cuda_funcs`` package, backed by the gfx950 HIP library.

An attention layer written against the reference API
(models/indexed_lattice_multi_head_attention_cuda.py:455-462,543-546) can import these instead and
run unchanged on one MI355X.  The kernels' compile-time constants, which the reference sets
globally through ``compile_kernels`` (models/cuda_funcs/kernel_manager.py:116-167), live in
``KernelManager`` here as well.
"""
from __future__ import annotations

import ctypes
import weakref
from typing import Optional

import torch

from . import _lib

CUPY_AVAILABLE = True   # name kept from the reference: "the native path is usable"


class KernelManager:
    """Global kernel constants (reference: models/cuda_funcs/kernel_manager.py:25-62,124-149)."""
    MAX_SYSTEM_SIZE: int = 320          # kept for API parity; these kernels have no size limit
    PE_THREAD_NUM: int = 64
    LATTICE_RANGE: int = 2
    MINIMUM_RANGE: int = 2
    SYMM_BREAK_NOISE: float = 1e-5
    NOISE_SEED: Optional[int] = None    # None: a fresh seed per call, as the reference draws one
    # a one-element int64 device tensor: mixed into the seed on the device and advanced after every
    # frame search, so that replays of a captured HIP graph (where NOISE_SEED is frozen) still draw
    # fresh noise
    NOISE_SEED_DEVICE: Optional[torch.Tensor] = None
    # options of this implementation (no reference counterpart)
    WINDOW_MODE: int = _lib.CFH_WINDOW_REFERENCE
    # distance window of the fused attention core (PeriodicAttentionCoreHIP).  Its angle encoding is the untruncated
    # Gaussian basis whatever this says; with the wide window (11 bins, +-5 sigma: a dropped bin is below 4e-6 of a
    # basis function's peak) the distance encoding is the untruncated basis as well to within that bound, i.e. the
    # core computes the reference's pure-PyTorch formulation
    # (models/indexed_lattice_multi_head_attention.py:580-588), which is what its results are held to (1e-4).
    # CFH_WINDOW_REFERENCE: the 9-bin window of the reference's CUDA kernels (+-4 sigma, dropped bin up to e^-8).
    CORE_WINDOW_MODE: int = _lib.CFH_WINDOW_WIDE
    # weight and bias gradients of the linear layers summed in a fixed order (per-workgroup partial tiles, added by
    # the last workgroup of a tile): the same bits from run to run.  False: float atomics, no scratch traffic.
    DETERMINISTIC_WEIGHT_GRADIENTS: bool = True
    # skip translations lighter than 2^-24 of their pair's heaviest: below the float32 resolution of the
    # normalised sum (measured on 256 crystals: every output within 1e-6 of the unpruned result); 0 keeps all
    PRUNE_LOG2: float = 24.0
    # keep the forward's window histograms (E,H,4,64 float32, 1 KB per (pair, head)) for the backward
    # pass, which then gathers only: about a third less backward time for 244 MB per layer at batch 256
    SAVE_HISTOGRAMS: bool = True
    # with the histograms kept: their weight gradients in a streaming kernel on a second stream of the
    # library beside the gather-only backward kernel (False: one kernel on the caller's stream)
    SECOND_STREAM: bool = True
    GRAD_COEF_QUIRK: bool = False
    # weight / bias gradients of the linear layers (leaf parameters): all layers of a backward pass in
    # one launch when the pass ends, instead of one launch per layer as the gradient is reached
    DEFER_WEIGHT_GRADS: bool = True
    # fused attention core: the weight gradients of the value encoding of all layers of a backward pass together when
    # the pass ends, instead of on the second stream beside every layer's main kernel, which they slow down by as
    # much as they gain there (False: inside every backward call)
    DEFER_CORE_WEIGHT_GRADS: bool = True
    COLLECT_STATS: bool = False         # count translations (read with _lib.read_stats)
    EVENT_LOG = None                    # a list: every library call appends (name, start, end) events
    _compiled_for = None


def compile_kernels(lattice_range: int, head_num: int, key_head_dim: int, value_pe_dim: int,
                    dim_angle_enc: int, value_head_dim: int, set_minimum_range: bool, cos_abs: int,
                    value_pe_dist_wscale: float, value_pe_angle_wscale: float,
                    value_pe_dist_coef: float, value_pe_angle_coef: float, symm_break_noise: float):
    """Same signature as the reference's run-time compiler.  The HIP kernels are built ahead of
    time, so this records the global constants and checks that the requested combination is among
    the compiled instantiations."""
    if key_head_dim != 16 or value_head_dim != 16:
        raise NotImplementedError(f"head dims ({key_head_dim},{value_head_dim}): only 16 is compiled")
    if value_pe_dim not in (0, 64) or dim_angle_enc not in (0, 16, 64):
        raise NotImplementedError(f"value_pe_dist_real={value_pe_dim}, value_pe_angle_real={dim_angle_enc}: "
                                  "compiled are 0 or 64 distance bins and 0, 16 or 64 angle bins")
    if value_pe_dim > 0 and not float(value_pe_dist_wscale) > 0.0:
        raise ValueError("value_pe_dist_wscale must be positive")
    if value_pe_dim > 0 and float(value_pe_dist_wscale) != 1.0 and dim_angle_enc == 16 and not _fused_core_default():
        # (kernels for a window width known at run time only exist for 0 and 64 angle bins in the two-step operators)
        raise NotImplementedError("value_pe_dist_wscale != 1 with 16 angle bins: only through the fused attention core")
    if dim_angle_enc == 64 and float(value_pe_angle_wscale) != 4.0:
        raise NotImplementedError("value_pe_angle_wscale: only 4.0 is compiled for 64 angle bins")
    if dim_angle_enc == 16 and float(value_pe_angle_wscale) < 1.0:
        # the 16-bin basis of the reference's lightweight setting (train_jarvis_time.sh:40-57) is evaluated whole,
        # as the reference does for it (its window leaves at most 7 bins out)
        raise NotImplementedError("value_pe_angle_wscale: at least 1.0 for 16 angle bins")
    KernelManager.LATTICE_RANGE = int(lattice_range)
    KernelManager.MINIMUM_RANGE = int(lattice_range) if set_minimum_range else 0
    KernelManager.SYMM_BREAK_NOISE = float(symm_break_noise)
    KernelManager._compiled_for = dict(head_num=head_num, cos_abs=cos_abs)
    _lib.load()


def _fused_core_default() -> bool:
    from . import attention
    return bool(attention.FUSED_CORE)


# --------------------------------------------------------------------------------------------------
def _params(H: int, Dh: int, K: int, A: int, cos_abs: int, dist_max: float, wscale: float,
            angle_wscale: float, dist_coef: float, angle_coef: float, cutoff_radius) -> _lib.CfhParams:
    p = _lib.CfhParams()
    p.struct_size = ctypes.sizeof(_lib.CfhParams)
    p.num_heads, p.head_dim, p.dist_bins, p.angle_bins = H, Dh, K, A
    p.cos_abs = int(cos_abs)
    p.lattice_range = KernelManager.LATTICE_RANGE
    p.minimum_range = KernelManager.MINIMUM_RANGE
    p.window_mode = KernelManager.WINDOW_MODE
    p.dist_max, p.dist_wscale, p.angle_wscale = float(dist_max), float(wscale), float(angle_wscale)
    p.dist_coef, p.angle_coef = float(dist_coef), float(angle_coef)
    p.cutoff_radius = 0.0 if cutoff_radius is None else float(cutoff_radius)
    p.prune_log2 = float(KernelManager.PRUNE_LOG2)
    p.symm_break_noise = float(KernelManager.SYMM_BREAK_NOISE)
    if KernelManager.NOISE_SEED is None:
        p.noise_seed = int(torch.randint(0, 2 ** 62, (1,)).item()) if p.symm_break_noise > 0 else 0
    else:
        p.noise_seed = int(KernelManager.NOISE_SEED)
    sd = KernelManager.NOISE_SEED_DEVICE
    p.noise_seed_dev = sd.data_ptr() if (sd is not None and p.symm_break_noise > 0) else None
    p.noise_seed_advance = 1          # every frame search advances the device word itself
    p.grad_coef_quirk = int(bool(KernelManager.GRAD_COEF_QUIRK))
    p.collect_stats = int(bool(KernelManager.COLLECT_STATS))
    p.flags = 0 if KernelManager.SECOND_STREAM else _lib.FLAG_SINGLE_STREAM
    return p


class _timed:
    """Brackets one library call with HIP events on the current stream when
    ``KernelManager.EVENT_LOG`` is a list; appends (name, start, end) to it."""

    def __init__(self, name, dev):
        self.name, self.dev, self.log = name, dev, KernelManager.EVENT_LOG

    def __enter__(self):
        if self.log is not None:
            self.start = torch.cuda.Event(enable_timing=True)
            self.end = torch.cuda.Event(enable_timing=True)
            self.start.record(torch.cuda.current_stream(self.dev))
        return self

    def __exit__(self, *exc):
        if self.log is not None:
            self.end.record(torch.cuda.current_stream(self.dev))
            self.log.append((self.name, self.start, self.end))
        return False


_edge_cache = {"ref": None, "version": None, "N": None, "val": None}


def seed_edge_schedule(edge_ij_e: torch.Tensor, e_start: torch.Tensor, order: torch.Tensor):
    """Hand over an (e_start, order) pair already known for ``edge_ij_e`` (geometry.py computes it)."""
    N = e_start.shape[0] - 1
    _edge_cache.update(ref=weakref.ref(edge_ij_e), version=edge_ij_e._version, N=N,
                       val=(e_start.contiguous(), order.to(torch.int32).contiguous()))


_atom_start_cache = {"ref": None, "version": None, "val": None}
_shift_table_cache = {"ref": None, "version": None, "table": None, "key": None}


def declare_shift_tables(tvecs_n: torch.Tensor):
    """Announce the lattice tensor that the layers of a forward pass share (the encoder does, once per pass): the
    first fused attention core of the pass fills a table of every crystal's translations sorted by length, the
    later ones and the backward pass read it instead of making it again."""
    _shift_table_cache.update(ref=weakref.ref(tvecs_n), version=tvecs_n._version, table=None, key=None)


def _shift_table_for(tvecs_n: torch.Tensor, tv: torch.Tensor, key, E: int):
    """(table, ready) for a fused-core call on lattices ``tv``: one buffer holding the sorted translations of every
    crystal (B,128,4) and, behind them, the nearest-image distances of every pair (E,2)."""
    c = _shift_table_cache
    nb = max(tv.shape[0], 1) * 512
    fresh = lambda: torch.empty(nb + 2 * max(E, 1), dtype=torch.float32, device=tv.device)
    key = key + (E,)
    if (c["ref"] is not None and c["ref"]() is tvecs_n and c["version"] == tvecs_n._version
            and tv.data_ptr() == tvecs_n.data_ptr()):
        if c["table"] is not None and c["key"] == key:
            return c["table"], 1
        table = fresh()
        c.update(table=table, key=key)
        return table, 0
    return fresh(), 0


def seed_atom_start(sizes: torch.Tensor, atom_start: torch.Tensor):
    """Hand over the (B+1) exclusive prefix sums already known for ``sizes`` (geometry.py computes them);
    the per-crystal mean of the same batch then needs no scan of its own."""
    _atom_start_cache.update(ref=weakref.ref(sizes), version=sizes._version, val=atom_start)


def edge_schedule(edge_ij_e: torch.Tensor, N: int):
    """(e_start (N+1) int64, order (N) int32) for an edge list whose edges are grouped by query atom.

    e_start is built as the reference's backward does (models/cuda_funcs/real_space_framed_proj.py:
    139-141); ``order`` lists atoms by descending neighbour count for the kernels' work queue.
    The result is cached for the last edge tensor seen (every layer of a forward pass shares it).
    """
    c = _edge_cache
    if c["ref"] is not None and c["ref"]() is edge_ij_e and c["version"] == edge_ij_e._version and c["N"] == N:
        return c["val"]
    cnt = torch.zeros(N + 1, dtype=torch.long, device=edge_ij_e.device)
    cnt.scatter_add_(0, edge_ij_e[0] + 1, torch.ones_like(edge_ij_e[0]))
    e_start = cnt.cumsum(0)
    order = torch.argsort(e_start[1:] - e_start[:-1], descending=True, stable=True).to(torch.int32)
    val = (e_start.contiguous(), order.contiguous())
    c.update(ref=weakref.ref(edge_ij_e), version=edge_ij_e._version, N=N, val=val)
    return val


def _f32c(t: Optional[torch.Tensor]) -> Optional[torch.Tensor]:
    if t is None:
        return None
    return t.detach().to(torch.float32).contiguous()


def _proj_weight(W: Optional[torch.Tensor], H: int, what: str) -> Optional[torch.Tensor]:
    """(1,H,Dh,bins) or (H,Dh,bins) -> contiguous (H,Dh,bins) (weights that differ from pair to pair are handled by
    the caller, see _weight_sets)."""
    if W is None:
        return None
    if W.dim() not in (3, 4):
        raise AssertionError(f"{what} must have 3 or 4 dimensions")
    if W.dim() == 4:
        if W.shape[0] != 1:
            raise NotImplementedError(f"{what}: only one shared projection (leading dim 1) is supported")
        W = W[0]
    if W.shape[0] != H:
        raise ValueError(f"{what}: expected {H} heads, got {W.shape[0]}")
    return _f32c(W)


def _frame_call(mode: int, q, k, a_ik, rpos_ij_e, tvecs_n, batch_i, edge_ij_e, frame1, rvlen_n,
                cutoff_radius):
    """mode 0: first axis (N,H,3); 1: second axis given the first; 2: orthonormal frames (3,N,H,3)."""
    second = mode == 1
    _lib.require_gpu(q, k, a_ik, rpos_ij_e, tvecs_n, batch_i, edge_ij_e)
    lib = _lib.load()
    N, H = a_ik.shape
    E = edge_ij_e.shape[1]
    Dh = q.shape[-1]
    dev = a_ik.device
    q, k, a = _f32c(q), _f32c(k), _f32c(a_ik)
    rpos, tv = _f32c(rpos_ij_e), _f32c(tvecs_n)
    rv = _f32c(rvlen_n)
    batch, edges = batch_i.contiguous(), edge_ij_e.contiguous()
    e_start, order = edge_schedule(edge_ij_e, N)
    out = torch.empty((3, N, H, 3) if mode == 2 else (N, H, 3), dtype=torch.float32, device=dev)
    p = _params(H, Dh, 0, 0, 0, 1.0, 1.0, 1.0, 1.0, 1.0, cutoff_radius if rv is not None else None)
    with torch.cuda.device(dev), _timed(("frame_axis1", "frame_axis2", "frame_axes")[mode], dev):
        need = lib.cfh_workspace_bytes(ctypes.byref(p), N, E)
        ws = _lib.workspace(dev, need)
        st = _lib.current_stream_ptr(dev)
        if mode == 2:
            rc = lib.cfh_frame_axes(ctypes.byref(p), _lib.ptr(q), _lib.ptr(k), _lib.ptr(a), _lib.ptr(rpos),
                                    _lib.ptr(tv), _lib.ptr(rv), _lib.ptr(batch), _lib.ptr(edges),
                                    _lib.ptr(e_start), _lib.ptr(order), N, E, tv.shape[0], _lib.ptr(out),
                                    _lib.ptr(ws), ws.numel(), st)
        elif not second:
            rc = lib.cfh_frame_axis1(ctypes.byref(p), _lib.ptr(q), _lib.ptr(k), _lib.ptr(a), _lib.ptr(rpos),
                                     _lib.ptr(tv), _lib.ptr(rv), _lib.ptr(batch), _lib.ptr(edges),
                                     _lib.ptr(e_start), _lib.ptr(order), N, E, tv.shape[0], _lib.ptr(out),
                                     _lib.ptr(ws), ws.numel(), st)
        else:
            f1 = _f32c(frame1)
            rc = lib.cfh_frame_axis2(ctypes.byref(p), _lib.ptr(q), _lib.ptr(k), _lib.ptr(a), _lib.ptr(rpos),
                                     _lib.ptr(tv), _lib.ptr(rv), _lib.ptr(batch), _lib.ptr(edges),
                                     _lib.ptr(e_start), _lib.ptr(order), _lib.ptr(f1), N, E, tv.shape[0],
                                     _lib.ptr(out), _lib.ptr(ws), ws.numel(), st)
    _lib.check(rc, ("cfh_frame_axis1", "cfh_frame_axis2", "cfh_frame_axes")[mode])
    return out


class ComputeFrame1MaximumMethodCUDA(torch.autograd.Function):
    """First frame axis (N,H,3).  Signature of models/cuda_funcs/calc_maximum_frame.py:24-91;
    ``v``, ``dist2_min_e``, ``K``, ``dist_max`` and ``wscale`` are unused there as well."""

    @staticmethod
    def forward(ctx, q, k, v, a_ik, rpos_ij_e, dist2_min_e, tvecs_n, batch_i, edge_ij_e, K, dist_max,
                wscale, rvlen_n=None, cutoff_radius=None):
        out = _frame_call(0, q, k, a_ik, rpos_ij_e, tvecs_n, batch_i, edge_ij_e, None, rvlen_n,
                          cutoff_radius)
        ctx.mark_non_differentiable(out)      # the reference returns None for every input gradient
        return out

    @staticmethod
    def backward(ctx, gframevec):
        return (None,) * 14


class ComputeFrame2MaximumMethodCUDA(torch.autograd.Function):
    """Second frame axis before orthogonalisation (N,H,3).  Signature of
    models/cuda_funcs/calc_maximum_frame.py:95-170."""

    @staticmethod
    def forward(ctx, q, k, v, a_ik, rpos_ij_e, dist2_min_e, tvecs_n, batch_i, edge_ij_e, K, dist_max,
                wscale, frame1, rvlen_n=None, cutoff_radius=None):
        out = _frame_call(1, q, k, a_ik, rpos_ij_e, tvecs_n, batch_i, edge_ij_e, frame1, rvlen_n,
                          cutoff_radius)
        ctx.mark_non_differentiable(out)
        return out

    @staticmethod
    def backward(ctx, gframevec):
        return (None,) * 15


class ComputeFramesMaximumMethodCUDA(torch.autograd.Function):
    """Orthonormal "max" frames (3,N,H,3) in one launch: both axis searches, Gram-Schmidt and the cross
    product of compute_frame_maximum_method_ (models/indexed_lattice_multi_head_attention_cuda.py:
    455-481).  No counterpart class in the reference; same leading arguments as the two above."""

    @staticmethod
    def forward(ctx, q, k, v, a_ik, rpos_ij_e, dist2_min_e, tvecs_n, batch_i, edge_ij_e, K, dist_max,
                wscale, rvlen_n=None, cutoff_radius=None):
        out = _frame_call(2, q, k, a_ik, rpos_ij_e, tvecs_n, batch_i, edge_ij_e, None, rvlen_n,
                          cutoff_radius)
        ctx.mark_non_differentiable(out)
        return out

    @staticmethod
    def backward(ctx, gframes):
        return (None,) * 14


def _stacked_frames(f1, f2, f3):
    """(3,N,H,3) contiguous float32 holding the three frames, without a copy when they already are
    the three slices of one such tensor."""
    base = f1._base
    if (base is not None and f2._base is base and f3._base is base and base.dtype == torch.float32
            and base.is_contiguous() and base.dim() == 4 and base.shape[0] == 3
            and f1.shape == base.shape[1:] and f1.data_ptr() == base.data_ptr()
            and f2.data_ptr() == base[1].data_ptr() and f3.data_ptr() == base[2].data_ptr()):
        return base.detach()
    return torch.stack([_f32c(f1), _f32c(f2), _f32c(f3)], 0).contiguous()


_PAIR_CHUNK = 4096      # pairs per step of the framework products below (bounds their temporaries)


def _weight_sets(W_k, E: int, N: int) -> str:
    """How the projection weights are shared (models/kernels/real_enc_frame_proj_fwd_length.cu:166-173):
    "shared" (leading dimension 1 or none), "edge" (one set per pair), "atom" (one set per query atom)."""
    if W_k is None or W_k.dim() == 3 or W_k.shape[0] == 1:
        return "shared"
    if W_k.shape[0] == E:
        return "edge"
    if W_k.shape[0] == N:
        return "atom"
    raise ValueError(f"W_k: leading dimension {W_k.shape[0]} is neither 1, the number of pairs {E} nor of atoms {N}")


def _pairwise_psi(Ws, coefs, rows, shat, Dh):
    """psi (E,H,Dh) = sum_enc coef_enc W_enc[rows[e]] . shat[e,:,enc] for weights that differ from pair to pair
    (``rows`` None: pair e uses set e).  Device products of the framework over the histograms the kernel made."""
    E, H = shat.shape[:2]
    out = torch.zeros((E, H, Dh), dtype=torch.float32, device=shat.device)
    for s0 in range(0, E, _PAIR_CHUNK):
        sl = slice(s0, min(E, s0 + _PAIR_CHUNK))
        for en, (W, c) in enumerate(zip(Ws, coefs)):
            if W is None:
                continue
            Wsel = W[sl] if rows is None else W[rows[sl]]
            out[sl] += c * torch.einsum("ehck,ehk->ehc", Wsel.to(torch.float32), shat[sl, :, en, :W.shape[-1]])
    return out


def _pairwise_backward(Ws, coefs, rows, shat, gpsi):
    """(g_pair (E,H,4,64), [gW_enc]) for upstream gpsi (E,H,Dh): the rows W^T gpsi the library's backward takes per
    pair, and the weight gradients gpsi (x) shat summed over the pairs of a weight set."""
    E, H = shat.shape[:2]
    g_pair = torch.zeros((E, H, 4, shat.shape[-1]), dtype=torch.float32, device=shat.device)
    gWs = [None if W is None else torch.zeros(W.shape, dtype=torch.float32, device=shat.device) for W in Ws]
    for s0 in range(0, E, _PAIR_CHUNK):
        sl = slice(s0, min(E, s0 + _PAIR_CHUNK))
        for en, (W, c) in enumerate(zip(Ws, coefs)):
            if W is None:
                continue
            bins = W.shape[-1]
            Wsel = (W[sl] if rows is None else W[rows[sl]]).to(torch.float32)
            g_pair[sl, :, en, :bins] = c * torch.einsum("ehck,ehc->ehk", Wsel, gpsi[sl])
            outer = c * torch.einsum("ehc,ehk->ehck", gpsi[sl], shat[sl, :, en, :bins])
            if rows is None:
                gWs[en][sl] = outer
            else:
                gWs[en].index_add_(0, rows[sl], outer)
    return g_pair, gWs


def _framed_pe_forward(ctx, qk, a_ik, rpos_ij_e, tvecs_n, batch_i, edge_ij_e, K, dist_max, wscale, W_k, W_k1,
                       W_k2, W_k3, frame_vecs, dim_angle_enc, value_pe_angle_scale, cos_abs, length_rbf_mul,
                       angle_rbf_mul, rvlen_n, cutoff_radius):
    """Forward of the two classes below.  ``qk``: None (``frame_vecs`` = the three frame tensors), or
    (q, k): the frames are searched in the same library call.  Returns (z, v or None, frames or None)."""
    _lib.require_gpu(a_ik, rpos_ij_e, tvecs_n, batch_i, edge_ij_e)
    lib = _lib.load()
    N, H = a_ik.shape
    E = edge_ij_e.shape[1]
    dev = a_ik.device
    K = int(K) if W_k is not None else 0
    sets = _weight_sets(W_k, E, N) if K > 0 else "shared"
    use_angle = K > 0 and W_k1 is not None and int(dim_angle_enc) > 0
    A = int(dim_angle_enc) if use_angle else 0
    pair_W = None
    if sets != "shared":
        # One weight set per pair or per query atom (W_num = E or N in the reference's kernels).  The kernels make z
        # and the histograms with the first set; psi and, in the backward, W^T gpsi and the weight gradients are
        # products of the framework over those histograms.
        if KernelManager.GRAD_COEF_QUIRK:
            raise NotImplementedError("GRAD_COEF_QUIRK with per-pair / per-atom projection weights")
        pair_W = [W_k] + ([W_k1, W_k2, W_k3] if use_angle else [None, None, None])
        for w in pair_W:
            if w is not None and (w.dim() != 4 or w.shape[0] != W_k.shape[0]):
                raise ValueError("per-pair / per-atom projection weights: every weight needs the same leading dimension")
        W_k, W_k1, W_k2, W_k3 = [None if w is None else w[:1] for w in pair_W]
    Wd = _proj_weight(W_k, H, "W_k") if K > 0 else None
    Wa = [_proj_weight(w, H, "W_k%d" % (n + 1)) for n, w in enumerate((W_k1, W_k2, W_k3))] if use_angle \
        else [None, None, None]
    Dh = Wd.shape[-2] if Wd is not None else 16
    a = _f32c(a_ik)
    rpos, tv, rv = _f32c(rpos_ij_e), _f32c(tvecs_n), _f32c(rvlen_n)
    batch, edges = batch_i.contiguous(), edge_ij_e.contiguous()
    e_start, order = edge_schedule(edge_ij_e, N)
    z = torch.empty((E, H), dtype=torch.float32, device=dev)
    v = torch.empty((E, H, Dh), dtype=torch.float32, device=dev) if K > 0 else None
    p = _params(H, Dh, K, A, cos_abs, float(dist_max), wscale, value_pe_angle_scale,
                length_rbf_mul, angle_rbf_mul, cutoff_radius if rv is not None else None)
    shat = None
    if K > 0 and (pair_W is not None or (KernelManager.SAVE_HISTOGRAMS and any(ctx.needs_input_grad))):
        shat = torch.empty((E, H, 4, K), dtype=torch.float32, device=dev)
    if qk is None:
        frames = _stacked_frames(*frame_vecs) if use_angle else None
        with torch.cuda.device(dev), _timed("framed_pe_forward", dev):
            ws = _lib.workspace(dev, lib.cfh_workspace_bytes(ctypes.byref(p), N, E))
            rc = lib.cfh_framed_pe_forward(
                ctypes.byref(p), _lib.ptr(a), _lib.ptr(rpos), _lib.ptr(tv), _lib.ptr(rv), _lib.ptr(batch),
                _lib.ptr(edges), _lib.ptr(e_start), _lib.ptr(order), _lib.ptr(Wd), _lib.ptr(Wa[0]),
                _lib.ptr(Wa[1]), _lib.ptr(Wa[2]), _lib.ptr(frames), N, E, tv.shape[0], _lib.ptr(z),
                _lib.ptr(v), None, _lib.ptr(shat), _lib.ptr(ws), ws.numel(), _lib.current_stream_ptr(dev))
        _lib.check(rc, "cfh_framed_pe_forward")
    else:
        _lib.require_gpu(*qk)
        q, k = _f32c(qk[0]), _f32c(qk[1])
        frames = torch.empty((3, N, H, 3), dtype=torch.float32, device=dev)
        with torch.cuda.device(dev), _timed("frame_axes_framed_pe_forward", dev):
            ws = _lib.workspace(dev, lib.cfh_workspace_bytes(ctypes.byref(p), N, E))
            rc = lib.cfh_frame_axes_framed_pe_forward(
                ctypes.byref(p), _lib.ptr(q), _lib.ptr(k), _lib.ptr(a), _lib.ptr(rpos), _lib.ptr(tv), _lib.ptr(rv),
                _lib.ptr(batch), _lib.ptr(edges), _lib.ptr(e_start), _lib.ptr(order), _lib.ptr(Wd), _lib.ptr(Wa[0]),
                _lib.ptr(Wa[1]), _lib.ptr(Wa[2]), N, E, tv.shape[0], _lib.ptr(frames), _lib.ptr(z), _lib.ptr(v),
                None, _lib.ptr(shat), _lib.ptr(ws), ws.numel(), _lib.current_stream_ptr(dev))
        _lib.check(rc, "cfh_frame_axes_framed_pe_forward")
    ctx.pairwise = None
    if pair_W is not None:
        rows = None if sets == "edge" else edges[0]
        coefs = (float(length_rbf_mul), float(angle_rbf_mul), float(angle_rbf_mul), float(angle_rbf_mul))
        v = _pairwise_psi([None if w is None else w.detach() for w in pair_W], coefs, rows, shat, Dh)
        ctx.pairwise = (sets, coefs)
        ctx.save_for_backward(a, rpos, tv, rv, batch, edges, e_start, order, *[None if w is None else w.detach() for w in pair_W],
                              frames if use_angle else None, z, shat)
        ctx.params = p
        ctx.w_shapes = [None if w is None else w.shape for w in pair_W]
        return z, v, frames
    ctx.save_for_backward(a, rpos, tv, rv, batch, edges, e_start, order, Wd, Wa[0], Wa[1], Wa[2],
                          frames if use_angle else None, z, shat)
    ctx.params = p
    ctx.w_shapes = [None if w is None else w.shape for w in (W_k, W_k1, W_k2, W_k3)]
    return z, v, frames


def _framed_pe_backward(ctx, gz_ek, gv_ekd):
    """ga (N,H) and the gradients of the four projection weights (in the shapes they came in)."""
    a, rpos, tv, rv, batch, edges, e_start, order, Wd, W1, W2, W3, frames, z, shat = ctx.saved_tensors
    lib = _lib.load()
    p = ctx.params
    N, H = a.shape
    E = edges.shape[1]
    dev = a.device
    gz = _f32c(gz_ek) if gz_ek is not None else torch.zeros_like(z)
    if getattr(ctx, "pairwise", None) is not None:
        sets, coefs = ctx.pairwise
        Ws = [Wd, W1, W2, W3]
        gpsi = _f32c(gv_ekd) if gv_ekd is not None else torch.zeros((E, H, Wd.shape[-2]), dtype=torch.float32, device=dev)
        g_pair, gWs = _pairwise_backward(Ws, coefs, None if sets == "edge" else edges[0], shat, gpsi)
        ga = torch.empty((N, H), dtype=torch.float32, device=dev)
        with torch.cuda.device(dev), _timed("framed_pe_backward", dev):
            ws = _lib.workspace(dev, lib.cfh_workspace_bytes(ctypes.byref(p), N, E))
            rc = lib.cfh_framed_pe_backward_pairwise(
                ctypes.byref(p), _lib.ptr(a), _lib.ptr(rpos), _lib.ptr(tv), _lib.ptr(rv), _lib.ptr(batch), _lib.ptr(edges),
                _lib.ptr(e_start), _lib.ptr(order), _lib.ptr(frames), _lib.ptr(z), _lib.ptr(gz), _lib.ptr(g_pair), N, E,
                tv.shape[0], _lib.ptr(ga), _lib.ptr(ws), ws.numel(), _lib.current_stream_ptr(dev))
        _lib.check(rc, "cfh_framed_pe_backward_pairwise")
        return ga, [g if g is None else g.to(w.dtype) for g, w in zip(gWs, Ws)]
    gv = None
    if Wd is not None:
        gv = _f32c(gv_ekd) if gv_ekd is not None else torch.zeros((E, H, Wd.shape[-2]), dtype=torch.float32, device=dev)
    ga = torch.empty((N, H), dtype=torch.float32, device=dev)
    gWd = torch.empty_like(Wd) if Wd is not None else None
    gWa = [torch.empty_like(w) if w is not None else None for w in (W1, W2, W3)]
    # The library runs this backward as a gather-only kernel here and a streaming kernel on its second stream.
    # The weight gradients of the linear layers collected so far (those of the layers behind this one) go to
    # that stream as well, behind the library's kernel, instead of waiting for the end of the pass; the join
    # is then made here.
    D = _DeferredWeightGrads
    second = (shat is not None and N > 0 and not (p.flags & _lib.FLAG_SINGLE_STREAM) and bool(D.pending)
              and D.task_id == torch._C._current_graph_task_id())
    flags = p.flags
    held = None
    with torch.cuda.device(dev):
        try:
            if second:
                p.flags = flags | _lib.FLAG_DEFER_JOIN
            with _timed("framed_pe_backward", dev):
                ws = _lib.workspace(dev, lib.cfh_workspace_bytes(ctypes.byref(p), N, E))
                rc = lib.cfh_framed_pe_backward(
                    ctypes.byref(p), _lib.ptr(a), _lib.ptr(rpos), _lib.ptr(tv), _lib.ptr(rv), _lib.ptr(batch),
                    _lib.ptr(edges), _lib.ptr(e_start), _lib.ptr(order), _lib.ptr(Wd), _lib.ptr(W1), _lib.ptr(W2),
                    _lib.ptr(W3), _lib.ptr(frames), _lib.ptr(z), _lib.ptr(gz), _lib.ptr(gv), _lib.ptr(shat), N, E,
                    tv.shape[0], _lib.ptr(ga), _lib.ptr(gWd), _lib.ptr(gWa[0]), _lib.ptr(gWa[1]), _lib.ptr(gWa[2]),
                    _lib.ptr(ws), ws.numel(), _lib.current_stream_ptr(dev))
            if second and rc == 0:
                held = D.flush(second_stream=True)
        finally:
            p.flags = flags
            if second:
                rcj = lib.cfh_second_stream_join(_lib.current_stream_ptr(dev))
    _lib.check(rc, "cfh_framed_pe_backward")
    if second:
        _lib.check(rcj, "cfh_second_stream_join")
    del held                # what the second stream read is ordered before everything that follows on this one
    gws = [g if g is None else g.reshape(s) for g, s in zip([gWd] + gWa, ctx.w_shapes)]
    return ga, gws


class RealEncodingWithFramedProjFuncCUDA(torch.autograd.Function):
    """z (E,H) and the framed value position encoding (E,H,Dh).  Signature and return convention of
    models/cuda_funcs/real_space_framed_proj.py:19-221: returns ``(z,)`` when ``K <= 0``, else
    ``(z, v)``; gradients flow to ``a_ik`` and the four projection weights only."""

    @staticmethod
    def forward(ctx, a_ik, rpos_ij_e, dist2_min_e, tvecs_n, batch_i, edge_ij_e, K, dist_max, wscale,
                W_k, W_k1, W_k2, W_k3, frame_vec_1, frame_vec_2, frame_vec_3, dim_angle_enc,
                value_pe_angle_scale, cos_abs, length_rbf_mul, angle_rbf_mul, rvlen_n=None,
                cutoff_radius=None):
        z, v, _ = _framed_pe_forward(ctx, None, a_ik, rpos_ij_e, tvecs_n, batch_i, edge_ij_e, K, dist_max, wscale,
                                     W_k, W_k1, W_k2, W_k3, (frame_vec_1, frame_vec_2, frame_vec_3),
                                     dim_angle_enc, value_pe_angle_scale, cos_abs, length_rbf_mul, angle_rbf_mul,
                                     rvlen_n, cutoff_radius)
        if v is None:
            return z,
        return z, v

    @staticmethod
    def backward(ctx, gz_ek, gv_ekd=None):
        ga, gws = _framed_pe_backward(ctx, gz_ek, gv_ekd)
        return (ga, None, None, None, None, None, None, None, None, gws[0], gws[1], gws[2], gws[3],
                None, None, None, None, None, None, None, None, None, None)


class RealEncodingWithMaxFramesFuncHIP(torch.autograd.Function):
    """The "max" frame search and RealEncodingWithFramedProjFuncCUDA behind it in one library call:
    (z, v, frames) with frames (3,N,H,3) as ComputeFramesMaximumMethodCUDA returns them (not
    differentiable).  ``q`` already divided by sqrt(Dh).  The remaining arguments are those of
    RealEncodingWithFramedProjFuncCUDA without the frames; needs the angle encoding (K > 0 and the three
    axis projections).  No counterpart class in the reference, which makes the two calls one after the
    other (models/indexed_lattice_multi_head_attention_cuda.py:666-734)."""

    @staticmethod
    def forward(ctx, q, k, a_ik, rpos_ij_e, dist2_min_e, tvecs_n, batch_i, edge_ij_e, K, dist_max, wscale,
                W_k, W_k1, W_k2, W_k3, dim_angle_enc, value_pe_angle_scale, cos_abs, length_rbf_mul,
                angle_rbf_mul, rvlen_n=None, cutoff_radius=None):
        if W_k is None or W_k1 is None or int(K) <= 0 or int(dim_angle_enc) <= 0:
            raise ValueError("RealEncodingWithMaxFramesFuncHIP needs the distance and the angle encoding")
        z, v, frames = _framed_pe_forward(ctx, (q, k), a_ik, rpos_ij_e, tvecs_n, batch_i, edge_ij_e, K, dist_max,
                                          wscale, W_k, W_k1, W_k2, W_k3, None, dim_angle_enc, value_pe_angle_scale,
                                          cos_abs, length_rbf_mul, angle_rbf_mul, rvlen_n, cutoff_radius)
        ctx.mark_non_differentiable(frames)
        ctx.set_materialize_grads(False)       # no zero tensor per pass for the gradient of the frames
        return z, v, frames

    @staticmethod
    def backward(ctx, gz_ek, gv_ekd=None, gframes=None):
        ga, gws = _framed_pe_backward(ctx, gz_ek, gv_ekd)
        return (None, None, ga, None, None, None, None, None, None, None, None, gws[0], gws[1], gws[2], gws[3],
                None, None, None, None, None, None, None)


# --------------------------------------------------------------------------------------------------
# consumers of z and psi.  Interim composites of stock PyTorch device ops with the reference's names
# and signatures; they run on the HIP device (no CPU path) but are not hand-written kernels yet.
# --------------------------------------------------------------------------------------------------
_layout_cache = {"ref": None, "version": None, "ok": None}


def declare_complete_blocks(edge_ij_e: torch.Tensor):
    """Record that ``edge_ij_e`` holds all n x n pairs of every crystal, sorted by i then j (true by
    construction for geometry.py), which spares the attention backward its one-off layout check."""
    _layout_cache.update(ref=weakref.ref(edge_ij_e), version=edge_ij_e._version, ok=True)


def _require_complete_blocks(edge_ij_e: torch.Tensor, e_start: torch.Tensor, N: int):
    c = _layout_cache
    if not (c["ref"] is not None and c["ref"]() is edge_ij_e and c["version"] == edge_ij_e._version):
        flag = torch.empty(1, dtype=torch.int32, device=edge_ij_e.device)
        lib = _lib.load()
        rc = lib.cfh_pair_layout_check(_lib.ptr(edge_ij_e), _lib.ptr(e_start), N, edge_ij_e.shape[1],
                                       _lib.ptr(flag), _lib.current_stream_ptr(edge_ij_e.device))
        _lib.check(rc, "cfh_pair_layout_check")
        c.update(ref=weakref.ref(edge_ij_e), version=edge_ij_e._version, ok=int(flag.item()) == 0)
    if not c["ok"]:
        raise ValueError("FusedDotProductAttentionCUDA.backward needs the complete n x n pair block of every "
                         "crystal, sorted by i then j (the layout the reference's irregular_transpose assumes)")


class FusedDotProductAttentionCUDA(torch.autograd.Function):
    """out_i = sum_j softmax_j(q_i.k_j + a_ij) (v_j + b_ij), per head, over the pairs of atom i.

    Signature and gradients of models/cuda_funcs/fused_dpa.py:17-170 (``que_ihk`` already divided by
    sqrt(Dh)).
    """

    @staticmethod
    def forward(ctx, que_ihk, key_ihk, val_ihk, aij_eh, bij_ehk, batch_i, edge_ij_e):
        _lib.require_gpu(que_ihk, key_ihk, val_ihk, aij_eh, bij_ehk, edge_ij_e)
        lib = _lib.load()
        N, H, K = que_ihk.shape
        E = edge_ij_e.shape[1]
        dev = que_ihk.device
        q, k, v = _f32c(que_ihk), _f32c(key_ihk), _f32c(val_ihk)
        a, b = _f32c(aij_eh), _f32c(bij_ehk)
        edge_c = edge_ij_e if edge_ij_e.is_contiguous() else edge_ij_e.contiguous()
        e_start, _ = edge_schedule(edge_ij_e, N)
        out = torch.empty((N, H, K), dtype=torch.float32, device=dev)
        prob = torch.empty((E, H), dtype=torch.float32, device=dev)
        with _timed("fused_dpa_forward", dev):
            rc = lib.cfh_fused_dpa_forward(_lib.ptr(q), _lib.ptr(k), _lib.ptr(v), _lib.ptr(a), _lib.ptr(b),
                                           _lib.ptr(edge_c), _lib.ptr(e_start), N, H, K, E, _lib.ptr(prob),
                                           _lib.ptr(out), _lib.current_stream_ptr(dev))
        _lib.check(rc, "cfh_fused_dpa_forward")
        ctx.save_for_backward(q, k, v, a, b, edge_c, e_start, prob, out)
        ctx.edge_ref = edge_ij_e
        ctx.in_dtype = que_ihk.dtype
        return out.to(que_ihk.dtype)

    @staticmethod
    def backward(ctx, go_ihk):
        q, k, v, a, b, edge_c, e_start, prob, out = ctx.saved_tensors
        lib = _lib.load()
        N, H, K = q.shape
        E = edge_c.shape[1]
        dev = q.device
        _require_complete_blocks(ctx.edge_ref, e_start, N)
        go = _f32c(go_ihk)
        gq, gk, gv = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)
        ga = torch.empty((E, H), dtype=torch.float32, device=dev)
        gb = torch.empty_like(b) if b is not None else None
        with _timed("fused_dpa_backward", dev):
            rc = lib.cfh_fused_dpa_backward(_lib.ptr(q), _lib.ptr(k), _lib.ptr(v), _lib.ptr(a), _lib.ptr(b),
                                            _lib.ptr(edge_c), _lib.ptr(e_start), _lib.ptr(prob), _lib.ptr(out),
                                            _lib.ptr(go), N, H, K, E, _lib.ptr(gq), _lib.ptr(gk), _lib.ptr(gv),
                                            _lib.ptr(ga), _lib.ptr(gb), _lib.current_stream_ptr(dev))
        _lib.check(rc, "cfh_fused_dpa_backward")
        dt = ctx.in_dtype
        return (gq.to(dt), gk.to(dt), gv.to(dt), ga.to(dt) if a is not None else None,
                gb.to(dt) if gb is not None else None, None, None)


class PeriodicAttentionCoreHIP(torch.autograd.Function):
    """The attention core of a layer in one library call:

        out_i = sum_j P_ij (v_j + psi_ij),   P_i. = softmax_j (qs_i . k_j + z_ij)

    with z and psi the lattice sums of RealEncodingWithFramedProjFuncCUDA and, when ``frames`` is None and the
    angle encoding is on, the "max" frames searched in the same call.  Returns ``(out (N,H,Dh), frames (3,N,H,3)
    or None)``; gradients flow to qs, k, v, a_ik and the four projection weights.  ``qs`` is the query already
    divided by sqrt(Dh).  Same result as RealEncodingWithMaxFramesFuncHIP followed by FusedDotProductAttentionCUDA
    (the reference's sequence, models/indexed_lattice_multi_head_attention_cuda.py:589-734 and :144-185), computed
    with one histogram per (atom, head) instead of one per (pair, head): psi (E,H,Dh) is never formed.  The angle
    encoding uses the full Gaussian basis (no +-4 sigma window: 64 bins as a 5-term series around the nearest bin,
    16 bins by adding all 16 basis values), the distance encoding the window of
    ``KernelManager.CORE_WINDOW_MODE``.  No counterpart class in the reference."""

    @staticmethod
    def supported(K, dim_angle_enc, wscale, angle_wscale, W_k, W_k1) -> bool:
        if W_k is None or int(K) != 64 or not float(wscale) > 0.0 or KernelManager.GRAD_COEF_QUIRK:
            return False
        if W_k.dim() == 4 and W_k.shape[0] != 1:
            return False
        A = int(dim_angle_enc) if W_k1 is not None else 0
        # 64 angle bins: moment series, accurate for sigma >= 3 bins; 16 bins (the lightweight setting): the whole
        # basis added directly, sigma >= 1 bin
        return A == 0 or (A == 64 and float(angle_wscale) >= 3.0) or (A == 16 and float(angle_wscale) >= 1.0)

    @staticmethod
    def forward(ctx, qs, k, v, a_ik, rpos_ij_e, tvecs_n, batch_i, edge_ij_e, K, dist_max, wscale, W_k, W_k1, W_k2,
                W_k3, dim_angle_enc, value_pe_angle_scale, cos_abs, length_rbf_mul, angle_rbf_mul, rvlen_n=None,
                cutoff_radius=None, frames=None):
        _lib.require_gpu(qs, k, v, a_ik, rpos_ij_e, tvecs_n, batch_i, edge_ij_e)
        lib = _lib.load()
        N, H = a_ik.shape
        E = edge_ij_e.shape[1]
        dev = a_ik.device
        use_angle = W_k1 is not None and int(dim_angle_enc) > 0
        A = int(dim_angle_enc) if use_angle else 0
        Wd = _proj_weight(W_k, H, "W_k")
        Wa = [_proj_weight(w, H, "W_k%d" % (n + 1)) for n, w in enumerate((W_k1, W_k2, W_k3))] if use_angle \
            else [None, None, None]
        Dh = Wd.shape[-2]
        q_, k_, v_, a = _f32c(qs), _f32c(k), _f32c(v), _f32c(a_ik)
        rpos, tv, rv = _f32c(rpos_ij_e), _f32c(tvecs_n), _f32c(rvlen_n)
        batch, edges = batch_i.contiguous(), edge_ij_e.contiguous()
        e_start, order = edge_schedule(edge_ij_e, N)
        _require_complete_blocks(edge_ij_e, e_start, N)
        p = _params(H, Dh, int(K), A, cos_abs, float(dist_max), wscale, value_pe_angle_scale, length_rbf_mul,
                    angle_rbf_mul, cutoff_radius if rv is not None else None)
        p.window_mode = int(KernelManager.CORE_WINDOW_MODE)
        hw = int(lib.cfh_fused_core_hist_words(ctypes.byref(p)))
        if hw <= 0:
            _lib.check(-1, "cfh_fused_core_hist_words")
        search = use_angle and frames is None
        if use_angle:
            fr = torch.empty((3, N, H, 3), dtype=torch.float32, device=dev) if search else _f32c(frames)
        else:
            fr = None
        z = torch.empty((E, H), dtype=torch.float32, device=dev)
        prob = torch.empty((E, H), dtype=torch.float32, device=dev)
        hist = torch.empty((H, N, hw), dtype=torch.float32, device=dev)      # head-major
        out = torch.empty((N, H, Dh), dtype=torch.float32, device=dev)
        # kept for the backward (and, the table, for the other layers of the pass): sorted translations of every
        # crystal, projection weights with the moment matrices folded in, item records
        table, table_ready = _shift_table_for(tvecs_n, tv, (p.lattice_range, p.minimum_range, p.cutoff_radius != 0.0,
                                                            rpos.data_ptr()), E)
        near_ptr = table.data_ptr() + 4 * 512 * max(tv.shape[0], 1)
        wcat = torch.empty((H, Dh, hw), dtype=torch.float32, device=dev)
        records = torch.empty((max(N, 1), H, 32), dtype=torch.int32, device=dev)
        cache = _lib.CfhCoreCache(table.data_ptr(), near_ptr, wcat.data_ptr(), records.data_ptr(), table_ready, 0, 0, 0)
        with torch.cuda.device(dev), _timed("fused_core_forward", dev):
            ws = _lib.workspace(dev, lib.cfh_fused_core_workspace_bytes(ctypes.byref(p), N, E, tv.shape[0], 0))
            rc = lib.cfh_fused_core_forward(
                ctypes.byref(p), _lib.ptr(q_), _lib.ptr(k_), _lib.ptr(v_), _lib.ptr(a), _lib.ptr(rpos), _lib.ptr(tv),
                _lib.ptr(rv), _lib.ptr(batch), _lib.ptr(edges), _lib.ptr(e_start), _lib.ptr(order), _lib.ptr(Wd),
                _lib.ptr(Wa[0]), _lib.ptr(Wa[1]), _lib.ptr(Wa[2]), N, E, tv.shape[0], _lib.ptr(fr), 1 if search else 0,
                _lib.ptr(z), _lib.ptr(prob), _lib.ptr(hist), _lib.ptr(out), ctypes.byref(cache), _lib.ptr(ws), ws.numel(),
                _lib.current_stream_ptr(dev))
        _lib.check(rc, "cfh_fused_core_forward")
        ctx.save_for_backward(q_, k_, v_, a, rpos, tv, rv, batch, edges, e_start, order, Wd, Wa[0], Wa[1], Wa[2], fr,
                              z, prob, hist, out, table, wcat, records)
        ctx.params = p
        ctx.w_shapes = [None if w is None else w.shape for w in (W_k, W_k1, W_k2, W_k3)]
        ctx.weights = (W_k, W_k1 if use_angle else None, W_k2 if use_angle else None, W_k3 if use_angle else None)
        ctx.in_dtype = qs.dtype
        if fr is not None:
            ctx.mark_non_differentiable(fr)
        ctx.set_materialize_grads(False)
        return out, fr

    @staticmethod
    def backward(ctx, gout, gframes=None):
        (q_, k_, v_, a, rpos, tv, rv, batch, edges, e_start, order, Wd, W1, W2, W3, fr, z, prob, hist,
         out, table, wcat, records) = ctx.saved_tensors
        lib = _lib.load()
        p = ctx.params
        N, H = a.shape
        E = edges.shape[1]
        dev = a.device
        go = _f32c(gout) if gout is not None else torch.zeros_like(out)
        gq, gk, gv = torch.empty_like(q_), torch.empty_like(k_), torch.empty_like(v_)
        ga = torch.empty((N, H), dtype=torch.float32, device=dev)
        glogit = torch.empty((E, H), dtype=torch.float32, device=dev)
        D = _DeferredWeightGrads
        if D.callback_queued and D.task_id != torch._C._current_graph_task_id():
            D.reset()                               # left over from a backward pass that raised
        # the weight gradients: with leaf parameters, zero-filled views of the pass's gradient arena that ONE library
        # call completes for all layers when the pass ends (see _DeferredWeightGrads); else made by this call
        defer_core = (KernelManager.DEFER_CORE_WEIGHT_GRADS and N > 0 and D.deferrable(*ctx.weights)
                      and all(w is None or (w.dtype == torch.float32 and w.numel() == Wd.numel()) for w in ctx.weights))
        if defer_core:
            views, refs = [], []
            for w in ctx.weights:
                if w is None:
                    views.append(None); refs.append(None)
                    continue
                views.append(D.take(w.numel(), dev))
                refs.append((D.arena, D.arena_off - ((w.numel() + 63) & ~63), w.numel()))
            gWd, gWa = views[0], views[1:]
            del views
        else:
            gWd = torch.empty_like(Wd)
            gWa = [torch.empty_like(w) if w is not None else None for w in (W1, W2, W3)]
        cache = _lib.CfhCoreCache(table.data_ptr(), None, wcat.data_ptr(), records.data_ptr(), 1, 1, 1, 0)
        # The library makes the weight gradients of the value encoding on its second stream, beside its main
        # kernel.  The weight gradients of the linear layers collected so far (those of the layers behind this one)
        # go to that stream as well instead of waiting for the end of the pass; the join is then made here.
        second = (N > 0 and not defer_core and not (p.flags & _lib.FLAG_SINGLE_STREAM) and bool(D.pending)
                  and D.task_id == torch._C._current_graph_task_id())
        flags = p.flags
        held = None
        rcj = 0
        with torch.cuda.device(dev):
            try:
                if defer_core:
                    p.flags = flags | _lib.FLAG_NO_WEIGHT_GRADS
                if second:
                    p.flags = flags | _lib.FLAG_DEFER_JOIN
                with _timed("fused_core_backward", dev):
                    ws = _lib.workspace(dev, lib.cfh_fused_core_workspace_bytes(ctypes.byref(p), N, E, tv.shape[0], 1))
                    rc = lib.cfh_fused_core_backward(
                        ctypes.byref(p), _lib.ptr(q_), _lib.ptr(k_), _lib.ptr(v_), _lib.ptr(a), _lib.ptr(rpos),
                        _lib.ptr(tv), _lib.ptr(rv), _lib.ptr(batch), _lib.ptr(edges), _lib.ptr(e_start), _lib.ptr(order),
                        _lib.ptr(Wd), _lib.ptr(W1), _lib.ptr(W2), _lib.ptr(W3), _lib.ptr(fr), _lib.ptr(z), _lib.ptr(prob),
                        _lib.ptr(hist), _lib.ptr(out), _lib.ptr(go), N, E, tv.shape[0], _lib.ptr(gq), _lib.ptr(gk),
                        _lib.ptr(gv), _lib.ptr(ga), _lib.ptr(glogit), *([None] * 4 if defer_core else
                                                                       [_lib.ptr(gWd), _lib.ptr(gWa[0]), _lib.ptr(gWa[1]),
                                                                        _lib.ptr(gWa[2])]),
                        ctypes.byref(cache), _lib.ptr(ws), ws.numel(), _lib.current_stream_ptr(dev))
                if second and rc == 0:
                    held = D.flush(second_stream=True)
            finally:
                p.flags = flags
                if second:
                    rcj = lib.cfh_second_stream_join(_lib.current_stream_ptr(dev))
        _lib.check(rc, "cfh_fused_core_backward")
        if second:
            _lib.check(rcj, "cfh_second_stream_join")
        del held            # what the second stream read is ordered before everything that follows on this one
        if defer_core:
            params_copy = _lib.CfhParams.from_buffer_copy(p)
            params_copy.flags = flags
            D.core_pending.append((params_copy, go, hist, N, refs, ctx.weights, [D.mark(w) if w is not None else None
                                                                                for w in ctx.weights]))
            if not D.callback_queued:
                torch.autograd.Variable._execution_engine.queue_callback(D.flush)
                D.callback_queued = True
                D.task_id = torch._C._current_graph_task_id()
        gws = [g if g is None else g.reshape(s) for g, s in zip([gWd] + gWa, ctx.w_shapes)]
        del gWd, gWa
        dt = ctx.in_dtype
        return (gq.to(dt), gk.to(dt), gv.to(dt), ga, None, None, None, None, None, None, None, gws[0], gws[1], gws[2],
                gws[3], None, None, None, None, None, None, None, None)


class IrregularMeanCUDA(torch.autograd.Function):
    """Per-crystal mean of per-atom features.  Signature of models/cuda_funcs/irregular_mean.py:19-70."""

    @staticmethod
    def forward(ctx, x_ik, batch_i, sizes):
        _lib.require_gpu(x_ik, batch_i)
        lib = _lib.load()
        dev = x_ik.device
        if sizes is None:
            B = int(batch_i.max().item()) + 1 if batch_i.numel() else 0
            sizes = torch.zeros(B, dtype=torch.long, device=dev)
            sizes.scatter_add_(0, batch_i, torch.ones_like(batch_i))
        B = sizes.shape[0]
        N = x_ik.shape[0]
        C = x_ik[0].numel() if N else int(torch.tensor(x_ik.shape[1:]).prod())
        c = _atom_start_cache
        if (c["ref"] is not None and c["ref"]() is sizes and c["version"] == sizes._version
                and c["val"].device == dev and c["val"].shape[0] == B + 1):
            atom_start = c["val"]
        else:
            atom_start = torch.nn.functional.pad(sizes.to(device=dev, dtype=torch.long).cumsum(0), (1, 0))
        x = _f32c(x_ik)
        out = torch.empty((B,) + tuple(x_ik.shape[1:]), dtype=torch.float32, device=dev)
        with _timed("crystal_mean_forward", dev):
            rc = lib.cfh_crystal_mean_forward(_lib.ptr(x), _lib.ptr(atom_start), N, B, C, _lib.ptr(out),
                                              _lib.current_stream_ptr(dev))
        _lib.check(rc, "cfh_crystal_mean_forward")
        ctx.save_for_backward(batch_i.contiguous(), atom_start)
        ctx.x_shape, ctx.in_dtype = tuple(x_ik.shape), x_ik.dtype
        return out.to(x_ik.dtype)

    @staticmethod
    def backward(ctx, gout):
        batch_i, atom_start = ctx.saved_tensors
        lib = _lib.load()
        dev = gout.device
        N = ctx.x_shape[0]
        B = atom_start.shape[0] - 1
        g = _f32c(gout)
        C = g[0].numel() if B else 0
        gx = torch.empty(ctx.x_shape, dtype=torch.float32, device=dev)
        with _timed("crystal_mean_backward", dev):
            rc = lib.cfh_crystal_mean_backward(_lib.ptr(g), _lib.ptr(batch_i), _lib.ptr(atom_start), N, B, C,
                                               _lib.ptr(gx), _lib.current_stream_ptr(dev))
        _lib.check(rc, "cfh_crystal_mean_backward")
        return gx.to(ctx.in_dtype), None, None


class _DeferredWeightGrads:
    """Weight and bias gradients of the linear layers of ONE backward pass, computed together.

    LinearHIP.backward hands autograd zero-filled gradient tensors (views of one arena that is cleared
    by a single fill) and records what has to be added to them; when the pass ends (a callback of the
    autograd engine) one call of cfh_linear_weight_bias_grad_batch adds x^T dy of every layer.  The
    gradients are complete when ``backward()`` / ``autograd.grad()`` return.  Only parameters that are
    leaves take part: nothing else reads their gradient before the pass ends.  If a parameter already
    had a ``.grad`` (accumulation over several passes), autograd has added the zeros to it at once and
    the batch call adds into that ``.grad`` instead.  A parameter with tensor hooks or post-accumulate hooks, or
    a pass with create_graph, is not deferred (``deferrable``): its products are made at once.  The batched
    kernel adds its row slices with float atomics, so the last bits of the weight gradients depend on the order
    in which the workgroups arrive: equal inputs give gradients equal to about 1e-7 relative, not bit for bit
    (``KernelManager.DEFER_WEIGHT_GRADS = False`` does not change that; the kernel is the same)."""
    ARENA_FLOATS = 1 << 21
    pending = []            # (x2, gy2, col0, O, dW ref, bias-gradient ref, weight, bias, marks)
    core_pending = []       # fused attention core: (params, gout, hist, N, gradient refs, weights, marks) per call
    arena = None
    arena_off = 0
    arenas = []             # keeps the gradient memory of the pass alive; the views themselves are NOT kept:
                            # autograd adopts a gradient tensor as .grad only if nobody else references it
    callback_queued = False
    task_id = -1            # autograd graph task the pending work belongs to

    @classmethod
    def take(cls, n: int, device) -> torch.Tensor:
        n_al = (n + 63) & ~63
        if cls.arena is None or cls.arena.device != device or cls.arena_off + n_al > cls.arena.numel():
            cls.arena = torch.zeros(max(cls.ARENA_FLOATS, n_al), dtype=torch.float32, device=device)
            cls.arena_off = 0
        v = cls.arena[cls.arena_off:cls.arena_off + n]
        cls.arena_off += n_al
        if not cls.arenas or cls.arenas[-1] is not cls.arena:
            cls.arenas.append(cls.arena)
        return v

    @staticmethod
    def mark(param):
        """The parameter's .grad tensor itself (kept alive, so that its identity cannot be reused by another
        tensor) and its version: ``changed`` tells whether autograd has set or added to .grad since."""
        g = param.grad
        return None if g is None else (g, g._version)

    @staticmethod
    def changed(param, mark) -> bool:
        g = param.grad
        if g is None or mark is None:
            return (g is None) != (mark is None)
        return g is not mark[0] or g._version != mark[1]

    @staticmethod
    def deferrable(*params) -> bool:
        """Deferring hands autograd zero-filled tensors that are completed when the pass ends.  That is only
        sound if nothing looks at a parameter's gradient before then: a float32 leaf without tensor hooks and
        without post-accumulate hooks (optimizer-in-backward, clipping in hooks), in a pass that does not
        build a graph of the backward itself (create_graph)."""
        if not KernelManager.DEFER_WEIGHT_GRADS or torch.is_grad_enabled():
            return False
        for w in params:
            if w is None:
                continue
            if not (w.is_leaf and w.dtype == torch.float32):
                return False
            if getattr(w, "_backward_hooks", None) or getattr(w, "_post_accumulate_grad_hooks", None):
                return False
        return True

    @classmethod
    def reset(cls):
        cls.pending = []
        cls.core_pending = []
        cls.arena = None
        cls.arena_off = 0
        cls.arenas = []
        cls.callback_queued = False

    @classmethod
    def flush(cls, second_stream=False):
        """All pending products in one launch.  ``second_stream``: now, on the library's second stream behind
        what a cfh_framed_pe_backward call that has just been made (with its join deferred) put there, beside
        that call's kernel on the current stream; the caller joins and keeps the list returned here -- the
        tensors the launch reads -- until then; the arena and the callback of the end of the pass stay as
        they are for the layers still to come.  At the end of the pass (``second_stream`` False) the weight
        gradients of the fused attention cores are made as well: one library call for all layers, behind the
        linear layers' launch."""
        pending, cls.pending = cls.pending, []
        core = []
        if not second_stream:
            core, cls.core_pending = cls.core_pending, []
            arenas, cls.arenas = cls.arenas, []
            cls.arena = None
            cls.arena_off = 0
            cls.callback_queued = False
        if not pending and not core:
            return None

        def view(ref):           # (arena, offset, count) -> tensor
            return ref[0][ref[1]:ref[1] + ref[2]]
        lib = _lib.load()
        dev = pending[0][1].device if pending else core[0][1].device
        jobs = (_lib.CfhLinearGradJob * max(len(pending), 1))()
        fixups = []
        for n, (x2, g2, col0, O, dW, db, weight, bias, w_mark, b_mark) in enumerate(pending):
            # dW, db: (arena, offset, count) of the zero-filled tensors handed to autograd (db: of the whole bias)
            # (x2 None: a sum over the rows of g2 alone, kept in the bias slots)
            dst_w = None if dW is None else dW[0].data_ptr() + 4 * dW[1]
            dst_b = None if db is None else db[0].data_ptr() + 4 * (db[1] + col0)
            wg = None if weight is None else weight.grad
            if wg is not None and cls.changed(weight, w_mark) and wg.data_ptr() != dst_w:
                # .grad was set or updated during this pass, but not by adopting our tensor: autograd
                # copied or accumulated it (adding our zeros), so the result belongs into .grad
                if wg.dtype == torch.float32 and wg.is_contiguous() and wg.device == dev:
                    dst_w = wg.data_ptr()
                else:
                    fixups.append((wg, view(dW).view(wg.shape)))
            if db is not None:
                bg = bias.grad
                if bg is not None and cls.changed(bias, b_mark) and bg.data_ptr() != db[0].data_ptr() + 4 * db[1]:
                    if bg.dtype == torch.float32 and bg.is_contiguous() and bg.device == dev:
                        dst_b = bg.data_ptr() + 4 * col0
                    elif col0 == 0:
                        fixups.append((bg, view(db)))
            J = jobs[n]
            J.x, J.dy = (None if x2 is None else x2.data_ptr()), g2.data_ptr() + 4 * col0
            J.dW, J.db = dst_w, dst_b
            if x2 is None:
                J.N, J.I, J.O, J.ldx, J.ldy = g2.shape[0], 1, O, 1, g2.stride(0)
            else:
                J.N, J.I, J.O, J.ldx, J.ldy = x2.shape[0], x2.shape[1], O, x2.stride(0), g2.stride(0)
        if second_stream:
            if fixups:                   # these need framework kernels on the current stream: at the end of the pass
                cls.pending = pending + cls.pending
                return None
            with torch.cuda.device(dev):
                side = ctypes.c_void_p()
                # no new fork: the stream was forked when the library call began, and what these jobs read
                # was complete before that
                _lib.check(lib.cfh_second_stream_get(ctypes.byref(side)), "cfh_second_stream_get")
                rc = _wgrad_batch(lib, jobs, len(pending), dev, side)
            _lib.check(rc, "cfh_linear_weight_bias_grad_batch")
            return pending
        # ---- the end of the pass
        groups = {}                      # calls of the core with the same constants share a library call
        for params, go, hist, N, refs, weights, marks in core:
            dst = []
            for ref, w, mark in zip(refs, weights, marks):
                if w is None:
                    dst.append(None)
                    continue
                d = ref[0].data_ptr() + 4 * ref[1]
                wg = w.grad
                if wg is not None and cls.changed(w, mark) and wg.data_ptr() != d:
                    if wg.dtype == torch.float32 and wg.is_contiguous() and wg.device == dev:
                        d = wg.data_ptr()
                    else:
                        fixups.append((wg, view(ref).view(wg.shape)))
                dst.append(d)
            groups.setdefault(bytes(params), (params, []))[1].append((go, hist, N, dst))
        # (one after the other on this stream: side by side on two streams the two launches took as long together
        # and the fork and join came on top)
        rc = rcc = 0
        with torch.cuda.device(dev):
            stream = _lib.current_stream_ptr(dev)
            if pending:
                with _timed("linear_weight_bias_grad_batch", dev):
                    rc = _wgrad_batch(lib, jobs, len(pending), dev, stream)
            for params, calls in groups.values():
                arr = (_lib.CfhCoreWgradJob * len(calls))()
                for J, (go, hist, N, dst) in zip(arr, calls):
                    J.gout, J.hist, J.N = go.data_ptr(), hist.data_ptr(), N
                    J.gW_dist, J.gW_axis1, J.gW_axis2, J.gW_axis3 = dst
                with _timed("fused_core_weight_gradients", dev):
                    ws = _lib.workspace(dev, lib.cfh_fused_core_weight_gradients_workspace_bytes(
                        ctypes.byref(params), len(calls)))
                    rcc = rcc or lib.cfh_fused_core_weight_gradients(ctypes.byref(params), arr, len(calls),
                                                                     _lib.ptr(ws), ws.numel(), stream)
        _lib.check(rc, "cfh_linear_weight_bias_grad_batch")
        _lib.check(rcc, "cfh_fused_core_weight_gradients")
        for grad, part in fixups:
            grad.add_(part.to(grad.dtype))
        return None


def _wgrad_batch(lib, jobs, njobs, dev, stream):
    """cfh_linear_weight_bias_grad_batch with the scratch that makes its sums run in a fixed order (the same bits
    from run to run); KernelManager.DETERMINISTIC_WEIGHT_GRADIENTS = False leaves the scratch out (float atomics)."""
    if not KernelManager.DETERMINISTIC_WEIGHT_GRADIENTS:
        return lib.cfh_linear_weight_bias_grad_batch(jobs, njobs, None, 0, stream)
    ws = _lib.wgrad_scratch(dev, stream, lib.cfh_linear_weight_bias_grad_batch_workspace_bytes(jobs, njobs))
    return lib.cfh_linear_weight_bias_grad_batch(jobs, njobs, _lib.ptr(ws), ws.numel(), stream)


def _linear_param_grads(x2, g2, weights, bias):
    """Gradients of y = x2 W^T + b (W the row-wise stack of ``weights``) for upstream g2: a list of
    weight gradients and the bias gradient (None without a bias).  For float32 leaf parameters the
    tensors returned are zero-filled views of the pass's gradient arena and the products are made by
    ONE library launch when the backward pass ends (see _DeferredWeightGrads); otherwise one launch
    here."""
    dev = x2.device
    I = x2.shape[1]
    O_all = g2.shape[1]
    x2 = _f32c(x2)
    g2 = _f32c(g2)
    D = _DeferredWeightGrads
    if D.callback_queued and D.task_id != torch._C._current_graph_task_id():
        D.reset()                               # left over from a backward pass that raised
    defer = D.deferrable(*weights, bias) and (bias is None or bias.dtype == torch.float32)
    if defer:
        def take(n):
            v = D.take(n, dev)
            return v, (D.arena, D.arena_off - ((n + 63) & ~63), n)
    else:
        total = sum(w.numel() for w in weights) + (O_all if bias is not None else 0)
        buf = torch.zeros(total, dtype=torch.float32, device=dev)
        state = [0]

        def take(n):
            v = buf[state[0]:state[0] + n]
            state[0] += n
            return v, (buf, state[0] - n, n)
    gb, gb_ref = take(O_all) if bias is not None else (None, None)
    gws, jobs, col0 = [], [], 0
    for w in weights:
        O = w.shape[0]
        dW, dW_ref = take(O * I)
        gws.append(dW.view(O, I))
        jobs.append((x2, g2, col0, O, dW_ref, gb_ref, w, bias,
                     D.mark(w) if defer else None, D.mark(bias) if defer and bias is not None else None))
        del dW
        col0 += O
    if defer:
        D.pending.extend(jobs)
        if not D.callback_queued:
            torch.autograd.Variable._execution_engine.queue_callback(D.flush)
            D.callback_queued = True
            D.task_id = torch._C._current_graph_task_id()
    else:
        lib = _lib.load()
        arr = (_lib.CfhLinearGradJob * len(jobs))()
        for n, (x2_, g2_, c0, O, dW, db, *_) in enumerate(jobs):
            J = arr[n]
            J.x, J.dy = x2_.data_ptr(), g2_.data_ptr() + 4 * c0
            J.dW = dW[0].data_ptr() + 4 * dW[1]
            J.db = None if db is None else db[0].data_ptr() + 4 * (db[1] + c0)
            J.N, J.I, J.O, J.ldx, J.ldy = x2_.shape[0], I, O, x2_.stride(0), g2_.stride(0)
        with torch.cuda.device(dev), _timed("linear_weight_bias_grad", dev):
            rc = _wgrad_batch(lib, arr, len(jobs), dev, _lib.current_stream_ptr(dev))
        _lib.check(rc, "cfh_linear_weight_bias_grad_batch")
    gws = [g.to(w.dtype) if g.dtype != w.dtype else g for g, w in zip(gws, weights)]
    gb_out = None if gb is None else (gb if gb.dtype == bias.dtype else gb.to(bias.dtype))
    return gws, gb_out


class LinearHIP(torch.autograd.Function):
    """y = x W^T + b, W the row-wise stack of ``weights`` (``stacked``: a tensor that already holds
    that stack, e.g. an alias of the parameters' shared storage; None: concatenated here).  Forward and
    input gradient are the framework's GEMMs; the weight and bias gradients come from the library: for
    leaf parameters deferred to one launch per backward pass (see _DeferredWeightGrads), otherwise
    one launch here.  Same values as torch.nn.functional.linear up to the order of the float32 sums."""

    SMALL_ROWS = 512        # up to this many rows the library's small-projection kernels replace the GEMMs

    @staticmethod
    def forward(ctx, x, bias, stacked, relu, *weights):
        if stacked is not None:
            W = stacked
        elif len(weights) == 1:
            W = weights[0]
        else:
            W = torch.cat(weights, dim=0)
        ctx.weights = weights
        ctx.bias = bias
        ctx.relu = bool(relu)
        rows = x.numel() // max(W.shape[1], 1)
        ctx.small = (0 < rows <= LinearHIP.SMALL_ROWS and x.dtype == torch.float32 and W.dtype == torch.float32
                     and (bias is None or bias.dtype == torch.float32))
        if ctx.small and W.shape[1] % 16 == 0:
            # few rows (one per crystal): the library's own kernel, which does not leave the product to
            # one or two workgroups
            lib = _lib.load()
            x2 = _f32c(x.reshape(rows, W.shape[1]))
            Wc = _f32c(W)
            bc = None if bias is None else _f32c(bias)
            y = torch.empty((rows, W.shape[0]), dtype=torch.float32, device=x.device)
            with torch.cuda.device(x.device), _timed("small_linear_forward", x.device):
                rc = lib.cfh_small_linear_forward(_lib.ptr(x2), _lib.ptr(Wc), _lib.ptr(bc), rows, W.shape[0], W.shape[1],
                                                  1 if relu else 0, _lib.ptr(y), _lib.current_stream_ptr(x.device))
            _lib.check(rc, "cfh_small_linear_forward")
            if x.dim() != 2:
                y = y.reshape(*x.shape[:-1], W.shape[0])
            if relu:
                ctx.save_for_backward(x, Wc, y)
            else:
                ctx.save_for_backward(x, Wc)
            return y
        if relu:
            # bias and rectifier in the epilogue of the library GEMM
            x2 = x.reshape(-1, W.shape[1])
            if bias is not None:
                y = torch._addmm_activation(bias.detach(), x2, W.detach().t(), use_gelu=False)
            else:
                y = torch.relu(x2.matmul(W.detach().t()))
            if x.dim() != 2:
                y = y.reshape(*x.shape[:-1], W.shape[0])
            ctx.save_for_backward(x, W.detach(), y)
            return y
        ctx.save_for_backward(x, W.detach())
        return torch.nn.functional.linear(x, W.detach(), None if bias is None else bias.detach())

    @staticmethod
    def backward(ctx, gy):
        if ctx.relu:
            x, W, y = ctx.saved_tensors
            gy = torch.ops.aten.threshold_backward(gy, y, 0.0)
        else:
            x, W = ctx.saved_tensors
        weights, bias = ctx.weights, ctx.bias
        gx = None
        if ctx.needs_input_grad[0]:
            if ctx.small and (W.shape[0] % 16 == 0 or W.shape[0] <= 64) and gy.dtype == torch.float32:
                lib = _lib.load()
                rows = gy.numel() // W.shape[0]
                g2c = _f32c(gy.reshape(rows, W.shape[0]))
                gx = torch.empty((rows, W.shape[1]), dtype=torch.float32, device=gy.device)
                with torch.cuda.device(gy.device), _timed("small_linear_dx", gy.device):
                    rc = lib.cfh_small_linear_dx(_lib.ptr(g2c), _lib.ptr(_f32c(W)), rows, W.shape[0], W.shape[1],
                                                 _lib.ptr(gx), _lib.current_stream_ptr(gy.device))
                _lib.check(rc, "cfh_small_linear_dx")
                gx = gx.reshape(x.shape)
            else:
                gx = gy.matmul(W)
        need_w = [ctx.needs_input_grad[4 + n] for n in range(len(weights))]
        need_b = bias is not None and ctx.needs_input_grad[1]
        if not (any(need_w) or need_b):
            return (gx, None, None, None) + (None,) * len(weights)
        gws, gb = _linear_param_grads(x.reshape(-1, W.shape[1]), gy.reshape(-1, W.shape[0]), weights, bias)
        return (gx, gb, None, None) + tuple(gws)


def linear(x: torch.Tensor, weight, bias: Optional[torch.Tensor] = None,
           stacked: Optional[torch.Tensor] = None, relu: bool = False) -> torch.Tensor:
    """torch.nn.functional.linear for device tensors with the library's weight-gradient kernel.
    ``weight``: a tensor (O,I), or a sequence of tensors (O_k,I) whose row-wise stack is the weight
    (``stacked``: that stack if it already exists in memory); ``relu``: max(0, .) of the result, in
    the epilogue of the GEMM."""
    weights = (weight,) if isinstance(weight, torch.Tensor) else tuple(weight)
    _lib.require_gpu(x, *weights)
    return LinearHIP.apply(x, bias, stacked, relu, *weights)


def _column_sum_grad(part, param):
    """Gradient of ``param`` (1-D, n elements) as the column sums of ``part`` (rows, n): for a float32 leaf a
    zero-filled view of the pass's gradient arena, filled by the weight-gradient launch at the end of the
    backward pass; otherwise summed at once."""
    n = part.shape[1]
    D = _DeferredWeightGrads
    if D.callback_queued and D.task_id != torch._C._current_graph_task_id():
        D.reset()                               # left over from a backward pass that raised
    if not (part.shape[0] > 0 and param is not None and param.dim() == 1 and D.deferrable(param)):
        return part.sum(0)
    g = D.take(n, part.device)
    ref = (D.arena, D.arena_off - ((n + 63) & ~63), n)
    D.pending.append((None, part, 0, n, None, ref, None, param, None, D.mark(param)))
    if not D.callback_queued:
        torch.autograd.Variable._execution_engine.queue_callback(D.flush)
        D.callback_queued = True
        D.task_id = torch._C._current_graph_task_id()
    return g


def _attention_inputs_grads(qkv, w, gs, consts, w_in, gqs, gk, gv, ga):
    """Backward of the attention inputs (see AttentionInputsHIP): the gradient of the stacked projection
    output and of the lattice weights ``w_in`` (for a float32 leaf: a zero-filled view of the pass's
    gradient arena, completed when the backward pass ends)."""
    H, Dh, c1, lb, c2, q_scale = consts
    lib = _lib.load()
    N = qkv.shape[0]
    gqs, gk, gv, ga = (None if g is None else _f32c(g) for g in (gqs, gk, gv, ga))
    gqkv = torch.empty_like(qkv)
    blocks = (N + 4 * (256 // (H * Dh)) - 1) // (4 * (256 // (H * Dh)))
    # scratch of the call: per-block partial sums of the weight gradient (256-byte aligned by the allocator)
    part = torch.empty((max(blocks, 1), H * Dh), dtype=torch.float32, device=qkv.device)
    D = _DeferredWeightGrads
    if D.callback_queued and D.task_id != torch._C._current_graph_task_id():
        D.reset()                               # left over from a backward pass that raised
    defer = N > 0 and w_in is not None and w_in.dim() == 1 and D.deferrable(w_in)
    if defer:
        # the column sums of the partials join the weight gradients of the pass in their one launch
        gw = D.take(H * Dh, qkv.device)
        gw_ref = (D.arena, D.arena_off - ((H * Dh + 63) & ~63), H * Dh)
    else:
        gw = torch.empty((H * Dh,), dtype=torch.float32, device=qkv.device)
    with _timed("attention_inputs_backward", qkv.device):
        rc = lib.cfh_attention_inputs_backward(_lib.ptr(qkv), _lib.ptr(w), _lib.ptr(gs), c1, lb, c2, q_scale,
                                               _lib.ptr(gqs), _lib.ptr(gk), _lib.ptr(gv), _lib.ptr(ga), N, H, Dh,
                                               _lib.ptr(gqkv), None if defer else _lib.ptr(gw), _lib.ptr(part),
                                               4 * part.numel(), _lib.current_stream_ptr(qkv.device))
    _lib.check(rc, "cfh_attention_inputs_backward")
    if defer:
        D.pending.append((None, part, 0, H * Dh, None, gw_ref, None, w_in, None, D.mark(w_in)))
        if not D.callback_queued:
            torch.autograd.Variable._execution_engine.queue_callback(D.flush)
            D.callback_queued = True
            D.task_id = torch._C._current_graph_task_id()
    return gqkv, gw


class AttentionInputsHIP(torch.autograd.Function):
    """(qs, k, v, a) from the stacked projection output qkv (N, 3 H Dh): query scaled by q_scale,
    key, value, and the Gaussian coefficient a (N,H) = ((1 - lb) elu(c1 alpha') + 1) c2 with
    alpha = q_h . lattice_w_h, alpha' = (alpha + gauss_scale[1]) gauss_scale[0] (gauss_scale None:
    alpha' = alpha; it is treated as a constant).  One launch each way instead of the framework's
    elementwise chain (reference arithmetic: models/indexed_lattice_multi_head_attention_cuda.py:896-940,
    query scaling :144-185)."""

    @staticmethod
    def supported(H: int, Dh: int) -> bool:
        return Dh == 16 and H >= 1 and 256 % (H * Dh) == 0

    @staticmethod
    def forward(ctx, qkv, lattice_w, gauss_scale, H, c1, lb, c2, q_scale):
        _lib.require_gpu(qkv, lattice_w)
        lib = _lib.load()
        N = qkv.shape[0]
        HD = qkv.shape[1] // 3
        Dh = HD // H
        qkv = _f32c(qkv)
        w = _f32c(lattice_w.detach())
        gs = _f32c(gauss_scale.detach()) if gauss_scale is not None else None
        qs = torch.empty((N, H, Dh), dtype=torch.float32, device=qkv.device)
        k = torch.empty_like(qs)
        v = torch.empty_like(qs)
        a = torch.empty((N, H), dtype=torch.float32, device=qkv.device)
        with _timed("attention_inputs_forward", qkv.device):
            rc = lib.cfh_attention_inputs_forward(_lib.ptr(qkv), _lib.ptr(w), _lib.ptr(gs), c1, lb, c2, q_scale, N, H, Dh,
                                                  _lib.ptr(qs), _lib.ptr(k), _lib.ptr(v), _lib.ptr(a),
                                                  _lib.current_stream_ptr(qkv.device))
        _lib.check(rc, "cfh_attention_inputs_forward")
        ctx.save_for_backward(qkv, w, gs)
        ctx.consts = (H, Dh, c1, lb, c2, q_scale)
        ctx.w_in = lattice_w
        ctx.set_materialize_grads(False)
        return qs, k, v, a

    @staticmethod
    def backward(ctx, gqs, gk, gv, ga):
        qkv, w, gs = ctx.saved_tensors
        gqkv, gw = _attention_inputs_grads(qkv, w, gs, ctx.consts, ctx.w_in, gqs, gk, gv, ga)
        return gqkv, gw, None, None, None, None, None, None


class LayerBridgeHIP(torch.autograd.Function):
    """Everything between the attention cores of two consecutive encoder layers in one launch (forward):

        x1 = x_res + attn Wo^T + bo,   h = relu(x1 W1^T + b1),   x2 = x1 + h W2^T + b2,

    and, when the weights of a next layer are given, qkv = x2 Wqkv^T + b_in and (qs, k, v, a) as
    AttentionInputsHIP makes them.  Returns ``(x2,)`` or ``(x2, qs, k, v, a)``.  ``stacked``: the three
    input-projection weights as one (3D, D) tensor if they share a storage, else None.  The backward
    pass uses the framework's GEMMs for the input gradients (the residual additions ride on them),
    the attention-inputs kernel, and the deferred weight-gradient launch.  For a layer without layer
    norm and dropout and with the ReLU activation; no counterpart class in the reference
    (models/indexed_latticeformer_encoder.py:606-648, models/indexed_lattice_multi_head_attention_cuda.py:
    399-409, 734, 896-940)."""

    FUSED_BACKWARD = True     # the four input-gradient products in one launch too (False: framework GEMMs)

    @staticmethod
    def backward_supported(D: int, F: int) -> bool:
        sl = lambda O: 1 if O // 64 >= 8 else 8 // (O // 64)
        part = max(sl(D) * 16 * (D + 4), sl(F) * 16 * (F + 4))
        return (16 * ((3 * D + 4) + 2 * (D + 4) + (F + 4)) + part) * 4 <= 160 * 1024

    @staticmethod
    def supported(D: int, F: int, H: int) -> bool:
        wide = max(F, 3 * D)
        return (D % 128 == 0 and F % 128 == 0 and D == 16 * H and H <= 32
                and (16 * (2 * (D + 4) + wide + 4) + 8 * 64 * 36) * 4 <= 160 * 1024)

    @staticmethod
    def forward(ctx, attn, x_res, Wo, bo, W1, b1, W2, b2, stacked, in_bias, lattice_w, gauss_scale, H, c1, lb,
                c2, q_scale, *qkv_weights):
        _lib.require_gpu(attn, x_res, Wo, W1, W2)
        lib = _lib.load()
        dev = attn.device
        N, D = attn.shape
        F = W1.shape[0]
        Dh = D // H
        has_next = len(qkv_weights) > 0
        attn_c, xres_c = _f32c(attn), _f32c(x_res)
        Wo_c, W1_c, W2_c = _f32c(Wo.detach()), _f32c(W1.detach()), _f32c(W2.detach())
        bo_c, b1_c, b2_c = (None if b is None else _f32c(b.detach()) for b in (bo, b1, b2))
        x1 = torch.empty((N, D), dtype=torch.float32, device=dev)
        h = torch.empty((N, F), dtype=torch.float32, device=dev)
        x2 = torch.empty((N, D), dtype=torch.float32, device=dev)
        Wq = bq = w = gs = qkv = qs = k = v = a = None
        if has_next:
            Wq = _f32c((stacked if stacked is not None else torch.cat(qkv_weights, dim=0)).detach())
            bq = None if in_bias is None else _f32c(in_bias.detach())
            w = _f32c(lattice_w.detach())
            gs = _f32c(gauss_scale.detach()) if gauss_scale is not None else None
            qkv = torch.empty((N, 3 * D), dtype=torch.float32, device=dev)
            qs = torch.empty((N, H, Dh), dtype=torch.float32, device=dev)
            k = torch.empty_like(qs)
            v = torch.empty_like(qs)
            a = torch.empty((N, H), dtype=torch.float32, device=dev)
        with torch.cuda.device(dev), _timed("layer_bridge_forward", dev):
            rc = lib.cfh_layer_bridge_forward(
                _lib.ptr(attn_c), _lib.ptr(xres_c), N, D, F, _lib.ptr(Wo_c), _lib.ptr(bo_c), _lib.ptr(W1_c),
                _lib.ptr(b1_c), _lib.ptr(W2_c), _lib.ptr(b2_c), _lib.ptr(Wq), _lib.ptr(bq), _lib.ptr(w), _lib.ptr(gs),
                float(c1), float(lb), float(c2), float(q_scale), H, _lib.ptr(x1), _lib.ptr(h), _lib.ptr(x2),
                _lib.ptr(qkv), _lib.ptr(qs), _lib.ptr(k), _lib.ptr(v), _lib.ptr(a), _lib.current_stream_ptr(dev))
        _lib.check(rc, "cfh_layer_bridge_forward")
        ctx.save_for_backward(attn_c, x1, h, x2, qkv, Wo_c, W1_c, W2_c, Wq, w, gs)
        ctx.params = (Wo, bo, W1, b1, W2, b2, tuple(qkv_weights), in_bias, lattice_w)
        ctx.consts = (H, Dh, c1, lb, c2, q_scale)
        ctx.set_materialize_grads(False)
        if has_next:
            return x2, qs, k, v, a
        return x2,

    @staticmethod
    def backward(ctx, g_x2, g_qs=None, g_k=None, g_v=None, g_a=None):
        attn, x1, h, x2, qkv, Wo_c, W1_c, W2_c, Wq, w, gs = ctx.saved_tensors
        Wo, bo, W1, b1, W2, b2, qkv_weights, in_bias, lattice_w = ctx.params
        n_fixed = 17
        g2 = None if g_x2 is None else _f32c(g_x2)
        g_in_bias = g_lw = gqkv = None
        g_qkv_w = [None] * len(qkv_weights)
        N, D = attn.shape
        F = W1_c.shape[0]
        dev = attn.device
        fused = LayerBridgeHIP.FUSED_BACKWARD and LayerBridgeHIP.backward_supported(D, F)
        with_inputs = bool(qkv_weights) and any(g is not None for g in (g_qs, g_k, g_v, g_a))
        if with_inputs and not fused:
            gqkv, g_lw = _attention_inputs_grads(qkv, w, gs, ctx.consts, lattice_w, g_qs, g_k, g_v, g_a)
        if g2 is None and not with_inputs:
            return (None,) * (n_fixed + len(qkv_weights))
        if fused:
            lib = _lib.load()
            ai = None
            keep = ()
            if with_inputs:
                # the backward of the attention inputs is made by the same launch
                H, Dh, c1, lb, c2, q_scale = ctx.consts
                gqkv = torch.empty((N, 3 * D), dtype=torch.float32, device=dev)
                part = torch.empty(((N + 15) // 16, D), dtype=torch.float32, device=dev)
                keep = tuple(None if g is None else _f32c(g) for g in (g_qs, g_k, g_v, g_a))
                adr = lambda t: None if t is None else t.data_ptr()
                ai = _lib.CfhAttentionInputsGrad(
                    adr(qkv), adr(w), adr(gs), adr(keep[0]), adr(keep[1]), adr(keep[2]), adr(keep[3]), adr(gqkv),
                    adr(part), float(c1), float(lb), float(c2), float(q_scale), H, 0)
            g2_out = torch.empty((N, D), dtype=torch.float32, device=dev) if with_inputs else None
            gh = torch.empty((N, F), dtype=torch.float32, device=dev)
            g1 = torch.empty((N, D), dtype=torch.float32, device=dev)
            g_attn = torch.empty((N, D), dtype=torch.float32, device=dev)
            with torch.cuda.device(dev), _timed("layer_bridge_backward", dev):
                rc = lib.cfh_layer_bridge_backward(_lib.ptr(g2), None, _lib.ptr(h), _lib.ptr(Wq), _lib.ptr(W2_c),
                                                   _lib.ptr(W1_c), _lib.ptr(Wo_c), N, D, F, _lib.ptr(g2_out), _lib.ptr(gh),
                                                   _lib.ptr(g1), _lib.ptr(g_attn),
                                                   None if ai is None else ctypes.byref(ai), _lib.current_stream_ptr(dev))
            _lib.check(rc, "cfh_layer_bridge_backward")
            del keep
            if with_inputs:
                g2 = g2_out
                g_lw = _column_sum_grad(part, lattice_w) if N > 0 else torch.zeros_like(w)
        else:
            if gqkv is not None:
                g2 = gqkv.matmul(Wq) if g2 is None else torch.addmm(g2, gqkv, Wq)
            gh = torch.ops.aten.threshold_backward(g2.matmul(W2_c), h, 0.0)
            g1 = torch.addmm(g2, gh, W1_c)
            g_attn = g1.matmul(Wo_c)
        if with_inputs:
            g_qkv_w, g_in_bias = _linear_param_grads(x2, gqkv, qkv_weights, in_bias)
        (gW2,), gb2 = _linear_param_grads(h, g2, (W2,), b2)
        (gW1,), gb1 = _linear_param_grads(x1, gh, (W1,), b1)
        (gWo,), gbo = _linear_param_grads(attn, g1, (Wo,), bo)
        return (g_attn, g1, gWo, gbo, gW1, gb1, gW2, gb2, None, g_in_bias, g_lw, None, None, None, None, None, None,
                *g_qkv_w)


