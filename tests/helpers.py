"""Shared builders of seeded test problems (CPU tensors; GPU tests move them to the device)."""
import math

import torch

from crystalframer_amd import synthetic
from oracle import torch_oracle as TO

H, DH, K, A = 8, 16, 64, 64
DIST_MAX = 14.0


class Problem:
    pass


def make_problem(num_crystals=6, atoms_lo=1, atoms_hi=5, len_lo=3.0, len_hi=8.0, ang_lo=70.0, ang_hi=110.0,
                 seed=0, alpha_std=1.0, dtype=torch.float64, w_scale=0.3):
    """Random crystals + random attention operands, all float64 on the CPU."""
    cb = synthetic.make_batch(num_crystals, atoms="uniform", atoms_lo=atoms_lo, atoms_hi=atoms_hi,
                              len_lo=len_lo, len_hi=len_hi, ang_lo=ang_lo, ang_hi=ang_hi, seed=seed)
    g = torch.Generator().manual_seed(seed + 1000)
    P = Problem()
    P.batch = cb.batch
    P.sizes = cb.sizes.tolist()
    # float32-representable inputs, held in float64 for the oracle
    P.pos = cb.pos.to(dtype)
    P.tvecs = cb.trans_vec.to(dtype)
    P.edges, P.rpos, recip, P.vcell = TO.geometry(P.pos, P.tvecs, P.sizes)
    P.rpos = P.rpos.float().to(dtype)
    P.rvlen = torch.norm(recip, 2, dim=-1).float().to(dtype)
    N = P.pos.shape[0]
    P.N, P.E = N, P.edges.shape[1]
    alpha = torch.randn(N, H, generator=g, dtype=torch.float64) * alpha_std
    P.a = TO.gaussian_coefficient(alpha).float().to(dtype)
    P.q = (torch.randn(N, H, DH, generator=g, dtype=torch.float64) / math.sqrt(DH)).float().to(dtype)
    P.k = torch.randn(N, H, DH, generator=g, dtype=torch.float64).float().to(dtype)
    P.v = torch.randn(N, H, DH, generator=g, dtype=torch.float64).float().to(dtype)
    P.W_k = (torch.randn(1, H, DH, K, generator=g, dtype=torch.float64) * w_scale).float().to(dtype)
    P.W_ax = [(torch.randn(1, H, DH, A, generator=g, dtype=torch.float64) * w_scale).float().to(dtype)
              for _ in range(3)]
    # random orthonormal frames (used when the test does not exercise frame selection)
    f1 = torch.nn.functional.normalize(torch.randn(N, H, 3, generator=g, dtype=torch.float64), dim=-1)
    f2 = torch.nn.functional.normalize(torch.randn(N, H, 3, generator=g, dtype=torch.float64), dim=-1)
    P.frames = [f.float().to(dtype) for f in TO.orthonormal_frame(f1, f2)]
    P.gz = torch.randn(P.E, H, generator=g, dtype=torch.float64).float().to(dtype)
    P.gpsi = torch.randn(P.E, H, DH, generator=g, dtype=torch.float64).float().to(dtype)
    return P


def rel_err(x, ref):
    """max |x-ref| / max |ref| (tensor-scale relative error)."""
    x, ref = x.detach(), ref.detach()
    scale = ref.abs().max().clamp_min(1e-30)
    return float((x.double().cpu() - ref.double().cpu()).abs().max() / scale.cpu())


def elem_err(x, ref, rtol=1e-4, atol_frac=1e-6):
    """Elementwise error in units of the allowance rtol*|ref| + atol_frac*max|ref|: the largest value of
    |x-ref| / (rtol*|ref| + atol_frac*max|ref|) over the tensor.  <= 1 means that every element is within
    ``rtol`` of its own reference value (small elements are given the absolute floor, a fraction
    ``atol_frac`` of the tensor's largest magnitude)."""
    x, ref = x.detach().double().cpu(), ref.detach().double().cpu()
    if ref.numel() == 0:
        return 0.0
    allow = rtol * ref.abs() + atol_frac * ref.abs().max().clamp_min(1e-30)
    return float(((x - ref).abs() / allow).max())


def problem_from_batch(cb, seed=9, w_scale=0.3):
    """Random attention operands (float64, CPU) for the crystals of a CrystalBatch."""
    gen = torch.Generator().manual_seed(seed)
    P = Problem()
    P.batch, P.sizes = cb.batch, cb.sizes.tolist()
    P.pos, P.tvecs = cb.pos.double(), cb.trans_vec.double()
    P.edges, P.rpos, recip, P.vcell = TO.geometry(P.pos, P.tvecs, P.sizes)
    P.rvlen = torch.norm(recip, 2, dim=-1)
    P.N, P.E = P.pos.shape[0], P.edges.shape[1]
    P.a = TO.gaussian_coefficient(torch.randn(P.N, H, generator=gen, dtype=torch.float64)).float().double()
    P.q = (torch.randn(P.N, H, DH, generator=gen, dtype=torch.float64) / 4).float().double()
    P.k = torch.randn(P.N, H, DH, generator=gen, dtype=torch.float64).float().double()
    P.v = torch.randn(P.N, H, DH, generator=gen, dtype=torch.float64).float().double()
    P.W_k = (torch.randn(1, H, DH, K, generator=gen, dtype=torch.float64) * w_scale).float().double()
    P.W_ax = [(torch.randn(1, H, DH, A, generator=gen, dtype=torch.float64) * w_scale).float().double()
              for _ in range(3)]
    f1 = torch.nn.functional.normalize(torch.randn(P.N, H, 3, generator=gen, dtype=torch.float64), dim=-1)
    f2 = torch.nn.functional.normalize(torch.randn(P.N, H, 3, generator=gen, dtype=torch.float64), dim=-1)
    P.frames = [f.float().double() for f in TO.orthonormal_frame(f1, f2)]
    return P


def first_crystals(P, nb):
    """The sub-problem made of the first ``nb`` crystals of P (operands sliced, weights shared)."""
    n_at, n_e = sum(P.sizes[:nb]), sum(s * s for s in P.sizes[:nb])
    S = Problem()
    S.sizes = P.sizes[:nb]
    S.N, S.E = n_at, n_e
    S.a, S.q, S.k, S.v = P.a[:n_at], P.q[:n_at], P.k[:n_at], P.v[:n_at]
    S.rpos, S.tvecs, S.batch, S.edges = P.rpos[:n_e], P.tvecs[:nb], P.batch[:n_at], P.edges[:, :n_e]
    S.rvlen, S.W_k, S.W_ax = P.rvlen[:nb], P.W_k, P.W_ax
    S.frames = [f[:n_at] for f in P.frames]
    return S


def check_model_gradients(model, leaves, auxes, n_at=None, tol=1e-4, min_checked=20):
    """Every parameter gradient of ``model`` (GPU) against the float64 leaves of the CPU model, and the gradients
    of the attention core's operands (scaled query, k, v, Gaussian coefficient) of every layer against the
    retained gradients of the CPU model's ``auxes``; ``n_at``: the CPU model ran on the first n_at atoms only.
    Tensor-scale bound ``tol`` and the element-wise bound |x - ref| <= tol |ref| + tol/10 max|ref|."""
    checked = 0
    for name, p in model.named_parameters():
        if p.grad is None:
            continue
        g_ref = leaves[name].grad
        assert g_ref is not None, name
        assert rel_err(p.grad, g_ref) < tol, (name, rel_err(p.grad, g_ref))
        assert elem_err(p.grad, g_ref, rtol=tol, atol_frac=tol / 10) <= 1.0, name
        checked += 1
    assert checked >= min_checked
    for li, (layer, aux) in enumerate(zip(model.encoder.layers, auxes)):
        sink = layer.self_attn.grad_sink
        for gpu_name, cpu_name in (("q", "qs"), ("k", "k"), ("v", "v"), ("a", "a")):
            got = sink[gpu_name] if n_at is None else sink[gpu_name][:n_at]
            ref = aux[cpu_name].grad
            assert rel_err(got, ref) < tol, (li, gpu_name, rel_err(got, ref))
            assert elem_err(got, ref, rtol=tol, atol_frac=tol / 10) <= 1.0, (li, gpu_name)
