"""Parity on the shapes of the other benchmark configurations: crystals with more than 64 atoms
(rows of pairs longer than one 64-lane block, configuration C4) and a large batch of small cells
with the distance encoding only (configuration C5).  Same tolerances as test_gpu_parity.py:
2e-5 forward, 5e-5 gradients against the float64 oracle with the same truncation windows."""
import pytest
import torch

import helpers as Hh
from oracle import c_oracle as CO
from oracle import torch_oracle as TO

pytestmark = pytest.mark.gpu

CUT = -3.5


def dev():
    return torch.device("cuda:0")


def g(t):
    return None if t is None else t.to(dtype=torch.float32, device=dev())


@pytest.fixture(autouse=True)
def _defaults():
    import crystalframer_amd as cf
    KM = cf.KernelManager
    saved = (KM.SYMM_BREAK_NOISE, KM.PRUNE_LOG2, KM.WINDOW_MODE)
    KM.SYMM_BREAK_NOISE, KM.PRUNE_LOG2, KM.WINDOW_MODE = 0.0, 24.0, 0
    yield
    KM.SYMM_BREAK_NOISE, KM.PRUNE_LOG2, KM.WINDOW_MODE = saved


def test_crystals_with_more_than_64_atoms():
    """Rows of 66-90 pairs: the second 64-pair block of a row, many groups per item, the long-row
    path of the frame search and of the attention kernels."""
    import crystalframer_amd as cf
    P = Hh.make_problem(num_crystals=2, atoms_lo=66, atoms_hi=90, len_lo=8.0, len_hi=14.0, ang_lo=70.0,
                        ang_hi=110.0, seed=301)
    assert max(P.sizes) > 64
    a = g(P.a).requires_grad_(True)
    Wk = g(P.W_k).requires_grad_(True)
    Wax = [g(w).requires_grad_(True) for w in P.W_ax]
    fr = [g(f) for f in P.frames]
    z, psi = cf.RealEncodingWithFramedProjFuncCUDA.apply(
        a, g(P.rpos), None, g(P.tvecs), P.batch.to(dev()), P.edges.to(dev()), 64, Hh.DIST_MAX, 1.0,
        Wk, Wax[0], Wax[1], Wax[2], fr[0], fr[1], fr[2], 64, 4.0, 0, 1.0, 1.0, g(P.rvlen), CUT)
    # the scalar C oracle in double precision (the tensor oracle needs minutes at this size)
    p = CO.make_params(cutoff_radius=CUT)
    zo, psio, _ = CO.pe_forward(p, P.a, P.rpos, P.tvecs, P.rvlen, P.batch, P.edges, P.W_k[0], P.W_ax, P.frames, "f64")
    assert Hh.rel_err(z, zo) < 2e-5
    assert Hh.rel_err(psi, psio) < 2e-5
    (z * g(P.gz)).sum().add((psi * g(P.gpsi)).sum()).backward()
    gao, gWdo, gWao = CO.pe_backward(p, P.a, P.rpos, P.tvecs, P.rvlen, P.batch, P.edges, P.W_k[0], P.W_ax, P.frames,
                                     zo, P.gz, P.gpsi, "f64")
    assert Hh.rel_err(a.grad, gao) < 5e-5
    assert Hh.rel_err(Wk.grad[0], gWdo) < 5e-5
    for ax in range(3):
        assert Hh.rel_err(Wax[ax].grad[0], gWao[ax]) < 5e-5

    # frames over rows longer than 64 pairs
    f1o, f2o = TO.frame_axes_max_vec(P.q, P.k, P.a, P.rpos, P.tvecs, P.batch, P.edges, rvlen=P.rvlen,
                                     cutoff_radius=CUT)
    args = (g(P.q), g(P.k), None, g(P.a), g(P.rpos), None, g(P.tvecs), P.batch.to(dev()), P.edges.to(dev()),
            64, Hh.DIST_MAX, 1.0, g(P.rvlen), CUT)
    frames = cf.ComputeFramesMaximumMethodCUDA.apply(*args)
    same1 = (frames[0].cpu().double() - f1o).abs().amax(-1) < 1e-5
    assert same1.double().mean() > 0.97          # the rest are float32 near-ties of the arg-max
    f2n = torch.nn.functional.normalize(f2o - (f1o * f2o).sum(-1, keepdim=True) * f1o, dim=-1)
    same2 = ((frames[1].cpu().double() - f2n).abs().amax(-1) < 1e-4) & same1
    assert same2.double().mean() > 0.94

    # attention over the same long rows
    gen = torch.Generator().manual_seed(9)
    zz = torch.randn(P.E, Hh.H, generator=gen, dtype=torch.float64)
    bb = torch.randn(P.E, Hh.H, Hh.DH, generator=gen, dtype=torch.float64)
    go = torch.randn(P.N, Hh.H, Hh.DH, generator=gen, dtype=torch.float64)
    l64 = [t.double().clone().requires_grad_(True) for t in (P.q, P.k, P.v, zz, bb)]
    o64, _ = TO.softmax_attention(*l64, P.batch, P.edges)
    (o64 * go).sum().backward()
    l32 = [g(t).requires_grad_(True) for t in (P.q, P.k, P.v, zz, bb)]
    o32 = cf.FusedDotProductAttentionCUDA.apply(*l32, P.batch.to(dev()), P.edges.to(dev()))
    (o32 * g(go)).sum().backward()
    assert Hh.rel_err(o32, o64) < 2e-5
    for x32, x64 in zip(l32, l64):
        assert Hh.rel_err(x32.grad, x64.grad) < 5e-5


def test_large_batch_of_small_cells_distance_encoding_only():
    """1024 crystals of 1-10 atoms, no angle encoding (A = 0): the first crystals of the batch
    against the oracle run on them alone, and the whole batch against itself split in two launches
    (an item's result must not depend on what else is in the batch)."""
    import crystalframer_amd as cf
    P = Hh.make_problem(num_crystals=1024, atoms_lo=1, atoms_hi=10, len_lo=3.0, len_hi=8.0, seed=302)

    def run(sl_atoms, sl_edges, sl_cry, atom0=0, cry0=0):
        a = g(P.a[sl_atoms]).requires_grad_(True)
        Wk = g(P.W_k).requires_grad_(True)
        edges = (P.edges[:, sl_edges] - atom0).to(dev()).contiguous()
        batch = (P.batch[sl_atoms] - cry0).to(dev())
        z, psi = cf.RealEncodingWithFramedProjFuncCUDA.apply(
            a, g(P.rpos[sl_edges]), None, g(P.tvecs[sl_cry]), batch, edges, 64, Hh.DIST_MAX, 1.0,
            Wk, None, None, None, None, None, None, 0, 4.0, 0, 1.0, 1.0, g(P.rvlen[sl_cry]), CUT)
        (z * g(P.gz[sl_edges])).sum().add((psi * g(P.gpsi[sl_edges])).sum()).backward()
        return z.detach(), psi.detach(), a.grad, Wk.grad

    full = slice(None)
    z, psi, ga, gW = run(full, full, full)
    assert torch.isfinite(z).all() and torch.isfinite(psi).all() and torch.isfinite(ga).all()

    # the first 12 crystals alone against the oracle
    nc = 12
    na = sum(P.sizes[:nc])
    ne = sum(s * s for s in P.sizes[:nc])
    ao = P.a[:na].clone().requires_grad_(True)
    Wko = P.W_k.clone().requires_grad_(True)
    zo, psio = TO.framed_pe(ao, P.rpos[:ne], P.tvecs[:nc], P.batch[:na], P.edges[:, :ne], Wko, None, None, K=64, A=0,
                            cos_abs=0, c_dist=1.0, c_angle=1.0, rvlen=P.rvlen[:nc], cutoff_radius=CUT,
                            windows="reference")
    (zo * P.gz[:ne]).sum().add((psio * P.gpsi[:ne]).sum()).backward()
    assert Hh.rel_err(z[:ne], zo) < 2e-5
    assert Hh.rel_err(psi[:ne], psio) < 2e-5
    assert Hh.rel_err(ga[:na], ao.grad) < 5e-5

    # two halves launched separately: outputs identical, weight gradients add up
    half_c = 512
    half_a = sum(P.sizes[:half_c])
    half_e = sum(s * s for s in P.sizes[:half_c])
    z1, psi1, ga1, gW1 = run(slice(0, half_a), slice(0, half_e), slice(0, half_c))
    z2, psi2, ga2, gW2 = run(slice(half_a, None), slice(half_e, None), slice(half_c, None), atom0=half_a, cry0=half_c)
    assert torch.equal(torch.cat([z1, z2]), z)
    assert torch.equal(torch.cat([psi1, psi2]), psi)
    assert Hh.rel_err(torch.cat([ga1, ga2]), ga) < 1e-6
    assert Hh.rel_err(gW1 + gW2, gW) < 1e-5


@pytest.mark.parametrize("num_crystals,atoms_hi", [(256, 40), (1500, 6), (3, 70), (1, 1)])
def test_geometry_launches_match_framework_expressions(num_crystals, atoms_hi):
    """cfh_crystal_geometry against the framework arithmetic it replaces: pairs, offsets and pair
    vectors exactly, the reciprocal lattice to float32 rounding, the work order as a permutation sorted by
    crystal size (ties in crystal order up to 1024 crystals, any order beyond)."""
    from crystalframer_amd import geometry, synthetic
    cb = synthetic.make_batch(num_crystals, atoms="uniform", atoms_lo=1, atoms_hi=atoms_hi, len_lo=3.0, len_hi=9.0,
                              ang_lo=65.0, ang_hi=115.0, seed=77).to(dev())
    geometry.USE_LIBRARY = False
    try:
        ref = geometry.crystal_geometry(cb.pos, cb.batch, cb.trans_vec, cb.sizes, cb.num_pairs)
    finally:
        geometry.USE_LIBRARY = True
    got = geometry.crystal_geometry(cb.pos, cb.batch, cb.trans_vec, cb.sizes, cb.num_pairs)
    assert got.num_edges == ref.num_edges == int((cb.sizes ** 2).sum())
    for name in ("edges", "e_start", "atom_start", "rpos"):
        assert torch.equal(getattr(got, name), getattr(ref, name)), name
    for name in ("vcell", "recip", "rvlen"):          # float32 rounding of the cross products may differ
        assert Hh.rel_err(getattr(got, name), getattr(ref, name)) < 1e-6, name
    n_of_atom = cb.sizes.to(dev())[cb.batch]
    order = got.order.long()
    assert torch.equal(torch.sort(order).values, torch.arange(order.numel(), device=dev()))
    assert (n_of_atom[order][:-1] >= n_of_atom[order][1:]).all()
    if num_crystals <= 1024:
        assert torch.equal(got.order, ref.order)
