"""Per-batch geometry shared by every attention layer of a forward pass.

Counterpart of ``compute_lattice_distances_for_cuda`` / ``get_edge_index``
(reference: models/indexed_latticeformer_encoder.py:15-44,175-245), restructured so that it runs on
the device without a Python loop over crystals: one host read (the edge count) per batch.
"""
from __future__ import annotations

import math
from dataclasses import dataclass
from typing import Optional

import torch


@dataclass
class CrystalGeometry:
    edges: torch.Tensor      # (2, E) int64, i-major: e = e_start[i] + j_local
    rpos: torch.Tensor       # (E, 3) float32  pos[j] - pos[i]
    recip: torch.Tensor      # (B, 3, 3) float32 reciprocal rows 2*pi*(t_b x t_c)/V
    rvlen: torch.Tensor      # (B, 3) float32 lengths of the reciprocal rows
    vcell: torch.Tensor      # (B,) float32 cell volume (signed determinant)
    e_start: torch.Tensor    # (N+1,) int64 first edge of each atom
    order: torch.Tensor      # (N,) int32 atoms sorted by descending crystal size (work-queue order)
    num_edges: int


def det_3x3(m: torch.Tensor) -> torch.Tensor:
    return (m[:, 0, 0] * m[:, 1, 1] * m[:, 2, 2] + m[:, 0, 1] * m[:, 1, 2] * m[:, 2, 0]
            + m[:, 0, 2] * m[:, 1, 0] * m[:, 2, 1] - m[:, 0, 2] * m[:, 1, 1] * m[:, 2, 0]
            - m[:, 0, 0] * m[:, 1, 2] * m[:, 2, 1] - m[:, 0, 1] * m[:, 1, 0] * m[:, 2, 2])


def reciprocal_vectors(trans: torch.Tensor):
    vcell = det_3x3(trans)
    recip = torch.stack([
        torch.linalg.cross(trans[:, 1], trans[:, 2], dim=1),
        torch.linalg.cross(trans[:, 2], trans[:, 0], dim=1),
        torch.linalg.cross(trans[:, 0], trans[:, 1], dim=1),
    ], dim=1) * (2.0 * math.pi / vcell[:, None, None])
    return recip.contiguous(), vcell.contiguous()


def edge_start_from_edges(edges: torch.Tensor, num_atoms: int) -> torch.Tensor:
    """(N+1,) first-edge offsets, as the reference's backward builds them
    (models/cuda_funcs/real_space_framed_proj.py:139-141)."""
    cnt = torch.zeros(num_atoms + 1, dtype=torch.long, device=edges.device)
    cnt.scatter_add_(0, edges[0] + 1, torch.ones_like(edges[0]))
    return cnt.cumsum(0)


def crystal_geometry(pos: torch.Tensor, batch: torch.Tensor, trans: torch.Tensor,
                     sizes: Optional[torch.Tensor] = None, num_edges: Optional[int] = None) -> CrystalGeometry:
    dev = pos.device
    B = trans.shape[0]
    N = pos.shape[0]
    if sizes is None:
        sizes = torch.zeros(B, dtype=torch.long, device=dev)
        sizes.scatter_add_(0, batch, torch.ones_like(batch))
    sizes = sizes.to(device=dev, dtype=torch.long)
    n_of_atom = sizes[batch]                                   # neighbours per atom
    atom_start = torch.cumsum(sizes, 0) - sizes                # first atom of each crystal
    e_start = torch.nn.functional.pad(torch.cumsum(n_of_atom, 0), (1, 0))
    if num_edges is not None:
        E = int(num_edges)
    else:
        E = int(e_start[-1].item()) if N > 0 else 0
    i_of_e = torch.repeat_interleave(torch.arange(N, device=dev), n_of_atom, output_size=E)
    j_of_e = atom_start[batch[i_of_e]] + (torch.arange(E, device=dev) - e_start[i_of_e])
    edges = torch.stack([i_of_e, j_of_e]).contiguous()
    rpos = (pos[j_of_e] - pos[i_of_e]).contiguous()
    recip, vcell = reciprocal_vectors(trans)
    rvlen = torch.norm(recip, 2, dim=-1).contiguous()
    order = torch.argsort(n_of_atom, descending=True, stable=True).to(torch.int32)
    return CrystalGeometry(edges, rpos, recip, rvlen, vcell, e_start, order, E)
