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


USE_LIBRARY = True       # device inputs with a known pair count: cfh_crystal_geometry instead of framework ops


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
    atom_start: Optional[torch.Tensor] = None   # (B+1,) int64 first atom of each crystal


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


def _crystal_geometry_hip(pos, batch, trans, sizes, num_edges: int) -> CrystalGeometry:
    """The same tensors from three launches of the library (cfh_crystal_geometry)."""
    from . import _lib
    lib = _lib.load()
    dev = pos.device
    N, B, E = pos.shape[0], trans.shape[0], int(num_edges)
    f32 = dict(dtype=torch.float32, device=dev)
    i64 = dict(dtype=torch.int64, device=dev)
    pos32 = pos.detach().to(torch.float32).contiguous()
    tv32 = trans.detach().to(torch.float32).contiguous()
    batch = batch.contiguous()
    edges = torch.empty((2, E), **i64)
    rpos = torch.empty((E, 3), **f32)
    recip = torch.empty((B, 3, 3), **f32)
    rvlen = torch.empty((B, 3), **f32)
    vcell = torch.empty((B,), **f32)
    e_start = torch.empty((N + 1,), **i64)
    atom_start = torch.empty((B + 1,), **i64)
    order = torch.empty((N,), dtype=torch.int32, device=dev)
    ws = torch.empty((2 * B + 1) * 8, dtype=torch.uint8, device=dev)
    with torch.cuda.device(dev):
        rc = lib.cfh_crystal_geometry(_lib.ptr(pos32), _lib.ptr(batch), _lib.ptr(tv32), _lib.ptr(sizes), N, B, E,
                                      _lib.ptr(edges), _lib.ptr(rpos), _lib.ptr(recip), _lib.ptr(rvlen), _lib.ptr(vcell),
                                      _lib.ptr(e_start), _lib.ptr(atom_start), _lib.ptr(order), _lib.ptr(ws), ws.numel(),
                                      _lib.current_stream_ptr(dev))
    _lib.check(rc, "cfh_crystal_geometry")
    return CrystalGeometry(edges, rpos, recip, rvlen, vcell, e_start, order, E, atom_start)


def crystal_geometry(pos: torch.Tensor, batch: torch.Tensor, trans: torch.Tensor,
                     sizes: Optional[torch.Tensor] = None, num_edges: Optional[int] = None) -> CrystalGeometry:
    """Device tensors with a known pair count go through the library; anything else (host tensors, a pair
    count that has to be read back) through the framework expressions below, which define the result."""
    dev = pos.device
    B = trans.shape[0]
    N = pos.shape[0]
    if sizes is None:
        sizes = torch.zeros(B, dtype=torch.long, device=dev)
        sizes.scatter_add_(0, batch, torch.ones_like(batch))
    sizes = sizes.to(device=dev, dtype=torch.long)
    if pos.is_cuda and num_edges is not None and USE_LIBRARY and pos.dtype == torch.float32 and batch.dtype == torch.int64:
        return _crystal_geometry_hip(pos, batch, trans, sizes.contiguous(), num_edges)
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
    return CrystalGeometry(edges, rpos, recip, rvlen, vcell, e_start, order, E,
                           torch.nn.functional.pad(torch.cumsum(sizes, 0), (1, 0)))
