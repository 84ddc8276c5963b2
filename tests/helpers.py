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
