"""Seeded synthetic crystal batches in the reference's input wire format.

Field layout follows dataloaders/dataset_latticeformer.py:32-37 of the reference:
``x (N,98)`` one-hot species, ``pos (N,3)`` Cartesian angstrom, ``trans_vec (B,3,3)`` rows =
lattice vectors, ``sizes (B)``, ``batch (N)``.
"""
from __future__ import annotations

import math
from dataclasses import dataclass
from typing import Optional

import torch

ATOM_FEAT_DIM = 98


@dataclass
class CrystalBatch:
    x: torch.Tensor          # (N, 98) float32 one-hot
    pos: torch.Tensor        # (N, 3) float32
    batch: torch.Tensor      # (N,) int64
    trans_vec: torch.Tensor  # (B, 3, 3) float32
    sizes: torch.Tensor      # (B,) int64
    num_pairs: int = -1      # sum of sizes^2, known on the host (spares the model a device read); -1: unknown
    zero_based: bool = False  # the caller knows that batch[0] == 0 (spares the model the subtraction of batch[0])

    def __post_init__(self):
        if self.num_pairs < 0 and not self.sizes.is_cuda:
            self.num_pairs = int((self.sizes.long() ** 2).sum())

    def to(self, device):
        return CrystalBatch(self.x.to(device), self.pos.to(device), self.batch.to(device),
                            self.trans_vec.to(device), self.sizes.to(device), self.num_pairs, self.zero_based)

    @property
    def num_crystals(self) -> int:
        return int(self.sizes.shape[0])


def lattice_from_parameters(lengths: torch.Tensor, angles_deg: torch.Tensor):
    """Rows = lattice vectors from (a,b,c,alpha,beta,gamma); also returns a validity mask."""
    a, b, c = lengths.unbind(-1)
    al, be, ga = (angles_deg * (math.pi / 180.0)).unbind(-1)
    ca, cb, cg, sg = torch.cos(al), torch.cos(be), torch.cos(ga), torch.sin(ga)
    zero = torch.zeros_like(a)
    v1 = torch.stack([a, zero, zero], -1)
    v2 = torch.stack([b * cg, b * sg, zero], -1)
    cy = (ca - cb * cg) / sg
    cz2 = 1.0 - cb * cb - cy * cy
    ok = cz2 > 1e-3
    cz = torch.sqrt(cz2.clamp_min(1e-3))
    v3 = torch.stack([c * cb, c * cy, c * cz], -1)
    return torch.stack([v1, v2, v3], -2), ok


def make_batch(num_crystals: int, *, atoms: str, atoms_lo: int, atoms_hi: int,
               len_lo: float, len_hi: float, ang_lo: float, ang_hi: float,
               seed: int = 123, lognormal_median: float = 8.0, lognormal_sigma: float = 0.6,
               species_hi: int = 94) -> CrystalBatch:
    """Draw one batch.  ``atoms`` is "uniform" or "lognormal" (median/sigma, clipped to lo..hi)."""
    g = torch.Generator().manual_seed(seed)
    if atoms == "uniform":
        sizes = torch.randint(atoms_lo, atoms_hi + 1, (num_crystals,), generator=g)
    elif atoms == "lognormal":
        z = torch.randn(num_crystals, generator=g, dtype=torch.float64)
        sizes = torch.round(torch.exp(math.log(lognormal_median) + lognormal_sigma * z))
        sizes = sizes.clamp(atoms_lo, atoms_hi).to(torch.long)
    else:
        raise ValueError(atoms)
    trans = torch.empty(num_crystals, 3, 3, dtype=torch.float64)
    todo = torch.ones(num_crystals, dtype=torch.bool)
    while bool(todo.any()):     # rejection: Gram determinant must be positive
        m = int(todo.sum())
        lengths = len_lo + (len_hi - len_lo) * torch.rand(m, 3, generator=g, dtype=torch.float64)
        angles = ang_lo + (ang_hi - ang_lo) * torch.rand(m, 3, generator=g, dtype=torch.float64)
        lat, ok = lattice_from_parameters(lengths, angles)
        idx = torch.nonzero(todo)[:, 0]
        trans[idx[ok]] = lat[ok]
        todo[idx[ok]] = False
    N = int(sizes.sum())
    batch = torch.repeat_interleave(torch.arange(num_crystals), sizes)
    frac = torch.rand(N, 3, generator=g, dtype=torch.float64)
    pos = torch.einsum("nd,ndx->nx", frac, trans[batch])
    species = torch.randint(1, species_hi + 1, (N,), generator=g)
    x = torch.zeros(N, ATOM_FEAT_DIM, dtype=torch.float32)
    x[torch.arange(N), species] = 1.0
    return CrystalBatch(x, pos.float(), batch, trans.float(), sizes, zero_based=True)


# The five benchmark configurations (batch shape only; the model settings live with the caller).
CONFIGS = {
    "C1": dict(num_crystals=16, atoms="uniform", atoms_lo=1, atoms_hi=8,
               len_lo=3.0, len_hi=10.0, ang_lo=70.0, ang_hi=110.0),
    "C2": dict(num_crystals=256, atoms="lognormal", atoms_lo=1, atoms_hi=60,
               len_lo=3.0, len_hi=12.0, ang_lo=60.0, ang_hi=120.0),
    "C3": dict(num_crystals=256, atoms="lognormal", atoms_lo=1, atoms_hi=60,
               len_lo=3.0, len_hi=12.0, ang_lo=60.0, ang_hi=120.0),
    "C4": dict(num_crystals=32, atoms="uniform", atoms_lo=40, atoms_hi=200,
               len_lo=8.0, len_hi=20.0, ang_lo=60.0, ang_hi=120.0),
    "C5": dict(num_crystals=4096, atoms="uniform", atoms_lo=1, atoms_hi=10,
               len_lo=3.0, len_hi=8.0, ang_lo=70.0, ang_hi=110.0),
}


def make_config(name: str, seed: int = 123, num_crystals: Optional[int] = None) -> CrystalBatch:
    kw = dict(CONFIGS[name])
    if num_crystals is not None:
        kw["num_crystals"] = num_crystals
    return make_batch(seed=seed, **kw)
