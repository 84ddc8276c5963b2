"""ctypes front end of the scalar C oracle (oracle/lattice_oracle.c).  TEST INFRASTRUCTURE ONLY.

``precision`` "f32" runs the reference's arithmetic (float, its loop order and truncation rules);
"f64" runs the same loops in double.  Tensors are CPU tensors; outputs come back in the working
precision.
"""
from __future__ import annotations

import ctypes
import math
import os
import subprocess

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
LIB = os.path.join(HERE, "liblattice_oracle.so")


class OrcParams(ctypes.Structure):
    _fields_ = [
        ("H", ctypes.c_int32), ("Dh", ctypes.c_int32), ("K", ctypes.c_int32), ("A", ctypes.c_int32),
        ("cos_abs", ctypes.c_int32), ("lattice_range", ctypes.c_int32), ("minimum_range", ctypes.c_int32),
        ("length_range", ctypes.c_int32), ("angle_range", ctypes.c_int32), ("cut_sigma", ctypes.c_int32),
        ("dist_max", ctypes.c_float), ("dist_wscale", ctypes.c_float), ("angle_sigma", ctypes.c_float),
        ("dist_coef", ctypes.c_float), ("angle_coef", ctypes.c_float), ("cutoff_radius", ctypes.c_float),
        ("grad_coef_quirk", ctypes.c_int32),
    ]


def build(force: bool = False) -> str:
    """Compile the oracle with gcc (oracle/Makefile)."""
    if force and os.path.exists(LIB):
        os.remove(LIB)
    res = subprocess.run(["make", "-C", HERE, "-s"], capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError("building the C oracle failed:\n" + res.stdout + res.stderr)
    return LIB


_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB):
            build()
        _lib = ctypes.CDLL(LIB)
    return _lib


def make_params(H=8, Dh=16, K=64, A=64, cos_abs=0, lattice_range=2, minimum_range=2, dist_max=14.0,
                dist_wscale=1.0, angle_wscale=4.0, dist_coef=1.0, angle_coef=1.0, cutoff_radius=-3.5,
                cut_sigma=4, windows="reference", grad_coef_quirk=False) -> OrcParams:
    p = OrcParams()
    p.H, p.Dh, p.K, p.A, p.cos_abs = H, Dh, K, A, cos_abs
    p.lattice_range, p.minimum_range, p.cut_sigma = lattice_range, minimum_range, cut_sigma
    if windows == "reference":
        # models/cuda_funcs/kernel_manager.py:146-147
        p.length_range = math.ceil(2 * dist_wscale * cut_sigma + 1)
        p.angle_range = math.ceil(2 * angle_wscale * cut_sigma + 1)
    elif windows == "full":
        p.length_range = p.angle_range = 0
    else:
        p.length_range, p.angle_range = windows
    p.dist_max, p.dist_wscale = dist_max, dist_wscale
    if A > 0:   # models/cuda_funcs/real_space_framed_proj.py:37-40
        p.angle_sigma = (angle_wscale / (A - 1)) if cos_abs else (2 * angle_wscale / (A - 1))
    p.dist_coef, p.angle_coef = dist_coef, angle_coef
    p.cutoff_radius = 0.0 if cutoff_radius is None else cutoff_radius
    p.grad_coef_quirk = int(grad_coef_quirk)
    return p


def _np(t, dt):
    if t is None:
        return None
    return np.ascontiguousarray(t.detach().cpu().numpy().astype(dt))


def _ptr(a):
    return None if a is None else a.ctypes.data_as(ctypes.c_void_p)


def _dt(precision):
    return {"f32": np.float32, "f64": np.float64}[precision]


def _stack_w(W_axes, dt):
    if W_axes is None:
        return None
    return np.ascontiguousarray(np.stack([_np(w, dt).reshape(w.shape[-3], w.shape[-2], w.shape[-1]) for w in W_axes]))


def _stack_f(frames, dt):
    if frames is None:
        return None
    return np.ascontiguousarray(np.stack([_np(f, dt) for f in frames]))


def e_start_of(edges: torch.Tensor, N: int) -> np.ndarray:
    cnt = torch.bincount(edges[0], minlength=N)
    return np.ascontiguousarray(np.concatenate([[0], np.cumsum(cnt.numpy())]).astype(np.int64))


def pe_forward(p: OrcParams, a, rpos, tvecs, rvlen, batch, edges, W_k, W_axes, frames, precision="f32"):
    dt = _dt(precision)
    N, H = a.shape
    E = edges.shape[1]
    a_, r_, t_ = _np(a, dt), _np(rpos, dt), _np(tvecs, dt)
    rv = _np(rvlen, np.float32)
    b_, e_ = _np(batch, np.int64), _np(edges, np.int64)
    Wd = _np(W_k, dt)
    Wa, fr = _stack_w(W_axes, dt), _stack_f(frames, dt)
    z = np.zeros((E, H), dt)
    psi = np.zeros((E, H, p.Dh), dt)
    d2min = np.zeros((E, H), dt)
    fn = getattr(lib(), "orc_pe_fwd_" + precision)
    fn.restype = None
    fn(ctypes.byref(p), _ptr(a_), _ptr(r_), _ptr(t_), _ptr(rv), _ptr(b_), _ptr(e_), ctypes.c_int64(N),
       ctypes.c_int64(E), _ptr(Wd), _ptr(Wa), _ptr(fr), _ptr(z), _ptr(psi), _ptr(d2min))
    return torch.from_numpy(z), torch.from_numpy(psi), torch.from_numpy(d2min)


def pe_backward(p: OrcParams, a, rpos, tvecs, rvlen, batch, edges, W_k, W_axes, frames, z, gz, gpsi,
                precision="f32"):
    dt = _dt(precision)
    N, H = a.shape
    E = edges.shape[1]
    a_, r_, t_ = _np(a, dt), _np(rpos, dt), _np(tvecs, dt)
    rv = _np(rvlen, np.float32)
    b_ = _np(batch, np.int64)
    es = e_start_of(edges, N)
    Wd = _np(W_k, dt)
    Wa, fr = _stack_w(W_axes, dt), _stack_f(frames, dt)
    z_, gz_, gp_ = _np(z, dt), _np(gz, dt), _np(gpsi, dt)
    ga = np.zeros((N, H), dt)
    gWd = np.zeros((H, p.Dh, p.K), dt) if Wd is not None else None
    gWa = np.zeros((3, H, p.Dh, p.A), dt) if Wa is not None else None
    fn = getattr(lib(), "orc_pe_bwd_" + precision)
    fn.restype = None
    fn(ctypes.byref(p), _ptr(a_), _ptr(r_), _ptr(t_), _ptr(rv), _ptr(b_), _ptr(es), ctypes.c_int64(N),
       ctypes.c_int64(E), _ptr(Wd), _ptr(Wa), _ptr(fr), _ptr(z_), _ptr(gz_), _ptr(gp_), _ptr(ga), _ptr(gWd),
       _ptr(gWa))
    t = torch.from_numpy
    return t(ga), (t(gWd) if gWd is not None else None), (t(gWa) if gWa is not None else None)


def frame_axes(p: OrcParams, q, k, a, rpos, tvecs, rvlen, batch, edges, precision="f32"):
    """(frame1, frame2max); q already divided by sqrt(Dh)."""
    dt = _dt(precision)
    N, H = a.shape
    E = edges.shape[1]
    q_, k_, a_, r_, t_ = _np(q, dt), _np(k, dt), _np(a, dt), _np(rpos, dt), _np(tvecs, dt)
    rv = _np(rvlen, np.float32)
    b_, e_ = _np(batch, np.int64), _np(edges, np.int64)
    f1 = np.zeros((N, H, 3), dt)
    f2 = np.zeros((N, H, 3), dt)
    fn1 = getattr(lib(), "orc_frame1_" + precision)
    fn2 = getattr(lib(), "orc_frame2_" + precision)
    fn1.restype = fn2.restype = None
    fn1(ctypes.byref(p), _ptr(q_), _ptr(k_), _ptr(a_), _ptr(r_), _ptr(t_), _ptr(rv), _ptr(b_), _ptr(e_),
        ctypes.c_int64(N), ctypes.c_int64(E), _ptr(f1))
    fn2(ctypes.byref(p), _ptr(q_), _ptr(k_), _ptr(a_), _ptr(r_), _ptr(t_), _ptr(rv), _ptr(b_), _ptr(e_),
        _ptr(f1), ctypes.c_int64(N), ctypes.c_int64(E), _ptr(f2))
    return torch.from_numpy(f1), torch.from_numpy(f2)


def dpa_forward(q, k, v, z, psi, edges, precision="f32"):
    dt = _dt(precision)
    N, H, Dh = q.shape
    E = edges.shape[1]
    q_, k_, v_, z_, p_ = _np(q, dt), _np(k, dt), _np(v, dt), _np(z, dt), _np(psi, dt)
    e_ = _np(edges, np.int64)
    es = e_start_of(edges, N)
    prob = np.zeros((E, H), dt)
    out = np.zeros((N, H, Dh), dt)
    fn = getattr(lib(), "orc_dpa_fwd_" + precision)
    fn.restype = None
    fn(ctypes.c_int(H), ctypes.c_int(Dh), _ptr(q_), _ptr(k_), _ptr(v_), _ptr(z_), _ptr(p_), _ptr(e_), _ptr(es),
       ctypes.c_int64(N), ctypes.c_int64(E), _ptr(prob), _ptr(out))
    return torch.from_numpy(out), torch.from_numpy(prob)


def dpa_backward(q, k, v, psi, edges, prob, out, gout, precision="f32"):
    dt = _dt(precision)
    N, H, Dh = q.shape
    E = edges.shape[1]
    q_, k_, v_, p_ = _np(q, dt), _np(k, dt), _np(v, dt), _np(psi, dt)
    e_ = _np(edges, np.int64)
    es = e_start_of(edges, N)
    pr, o_, go = _np(prob, dt), _np(out, dt), _np(gout, dt)
    gq, gk, gv = (np.zeros((N, H, Dh), dt) for _ in range(3))
    gz = np.zeros((E, H), dt)
    gpsi = np.zeros((E, H, Dh), dt) if p_ is not None else None
    fn = getattr(lib(), "orc_dpa_bwd_" + precision)
    fn.restype = None
    fn(ctypes.c_int(H), ctypes.c_int(Dh), _ptr(q_), _ptr(k_), _ptr(v_), _ptr(p_), _ptr(e_), _ptr(es),
       ctypes.c_int64(N), ctypes.c_int64(E), _ptr(pr), _ptr(o_), _ptr(go), _ptr(gq), _ptr(gk), _ptr(gv),
       _ptr(gz), _ptr(gpsi))
    t = torch.from_numpy
    return t(gq), t(gk), t(gv), t(gz), (t(gpsi) if gpsi is not None else None)


def crystal_mean(x, sizes, precision="f32"):
    dt = _dt(precision)
    x_ = _np(x, dt)
    start = np.ascontiguousarray(np.concatenate([[0], np.cumsum(np.asarray(sizes))]).astype(np.int64))
    B = len(sizes)
    D = x_.size // x_.shape[0]
    out = np.zeros((B, D), dt)
    fn = getattr(lib(), "orc_crystal_mean_" + precision)
    fn.restype = None
    fn(_ptr(x_), _ptr(start), ctypes.c_int64(B), ctypes.c_int64(D), _ptr(out))
    return torch.from_numpy(out).reshape((B,) + tuple(x.shape[1:]))
