"""The two large benchmark configurations at their full sizes: the large-cell stress case (32 crystals
of 40-200 atoms, about half a million pairs, one max-frame layer forward + backward) and the inference
batch (4096 small crystals, 4-layer encoder forward, with and without the angle encoding).  At these
sizes the oracle is too slow for the whole batch, so the checks are properties that do not depend on
the size -- a crystal's results do not depend on what else is in the batch, the backward pass is linear
in the upstream gradients, rotation leaves z and psi unchanged, reordering the crystals reorders the
outputs -- plus the scalar port of the reference kernels on one crystal of the batch."""
import pytest
import torch

import helpers as Hh
from oracle import c_oracle as CO
from oracle import torch_oracle as TO

pytestmark = pytest.mark.gpu

CUT = -3.5


@pytest.fixture(autouse=True)
def _defaults():
    import crystalframer_amd as cf
    KM = cf.KernelManager
    saved = (KM.SYMM_BREAK_NOISE, KM.PRUNE_LOG2, KM.WINDOW_MODE, KM.GRAD_COEF_QUIRK, KM.LATTICE_RANGE, KM.MINIMUM_RANGE,
             KM.SAVE_HISTOGRAMS)
    KM.SYMM_BREAK_NOISE = 0.0
    KM.PRUNE_LOG2 = 24.0
    KM.WINDOW_MODE = 0
    KM.GRAD_COEF_QUIRK = False
    KM.LATTICE_RANGE, KM.MINIMUM_RANGE = 2, 2
    yield
    (KM.SYMM_BREAK_NOISE, KM.PRUNE_LOG2, KM.WINDOW_MODE, KM.GRAD_COEF_QUIRK, KM.LATTICE_RANGE, KM.MINIMUM_RANGE,
     KM.SAVE_HISTOGRAMS) = saved


def dev():
    return torch.device("cuda:0")


def g(t):
    return None if t is None else t.to(dtype=torch.float32, device=dev())


def _large_cell_problem():
    from crystalframer_amd import synthetic
    cb = synthetic.make_config("C4", seed=123)
    gen = torch.Generator().manual_seed(41)
    P = Hh.Problem()
    P.batch, P.sizes = cb.batch, cb.sizes.tolist()
    P.pos, P.tvecs = cb.pos.double(), cb.trans_vec.double()
    P.edges, P.rpos, recip, _ = TO.geometry(P.pos, P.tvecs, P.sizes)
    P.rpos = P.rpos.float().double()
    P.rvlen = torch.norm(recip, 2, dim=-1).float().double()
    P.N, P.E = P.pos.shape[0], P.edges.shape[1]
    f32 = lambda t: t.float().double()
    P.a = f32(TO.gaussian_coefficient(torch.randn(P.N, Hh.H, generator=gen, dtype=torch.float64)))
    P.q = f32(torch.randn(P.N, Hh.H, Hh.DH, generator=gen, dtype=torch.float64) / 4)
    P.k = f32(torch.randn(P.N, Hh.H, Hh.DH, generator=gen, dtype=torch.float64))
    P.W_k = f32(torch.randn(1, Hh.H, Hh.DH, 64, generator=gen, dtype=torch.float64) * 0.3)
    P.W_ax = [f32(torch.randn(1, Hh.H, Hh.DH, 64, generator=gen, dtype=torch.float64) * 0.3) for _ in range(3)]
    return P


def _slice_crystal(P, b):
    """Atoms, pairs and lattice of crystal b as a problem of its own."""
    a0 = sum(P.sizes[:b])
    e0 = sum(s * s for s in P.sizes[:b])
    n = P.sizes[b]
    S = Hh.Problem()
    S.sl_a, S.sl_e = slice(a0, a0 + n), slice(e0, e0 + n * n)
    S.a, S.q, S.k = P.a[S.sl_a], P.q[S.sl_a], P.k[S.sl_a]
    S.rpos, S.edges = P.rpos[S.sl_e], P.edges[:, S.sl_e] - a0
    S.batch = torch.zeros(n, dtype=torch.long)
    S.tvecs, S.rvlen = P.tvecs[b:b + 1], P.rvlen[b:b + 1]
    S.W_k, S.W_ax = P.W_k, P.W_ax
    S.N, S.E, S.sizes = n, n * n, [n]
    return S


def _layer(P, gz, gpsi):
    """Frame search, then the lattice sums forward and backward, through the operator boundary."""
    import crystalframer_amd as cf
    a = g(P.a).requires_grad_(True)
    Wk = g(P.W_k).requires_grad_(True)
    Wax = [g(w).requires_grad_(True) for w in P.W_ax]
    rpos, tv, rv = g(P.rpos), g(P.tvecs), g(P.rvlen)
    batch, edges = P.batch.to(dev()), P.edges.to(dev()).contiguous()
    q, k = g(P.q), g(P.k)
    f1 = cf.ComputeFrame1MaximumMethodCUDA.apply(q, k, None, a.detach(), rpos, None, tv, batch, edges, 64,
                                                 Hh.DIST_MAX, 1.0, rv, CUT)
    f2 = cf.ComputeFrame2MaximumMethodCUDA.apply(q, k, None, a.detach(), rpos, None, tv, batch, edges, 64,
                                                 Hh.DIST_MAX, 1.0, f1, rv, CUT)
    fr = [f.float().to(dev()) for f in TO.orthonormal_frame(f1.double(), f2.double())]
    z, psi = cf.RealEncodingWithFramedProjFuncCUDA.apply(
        a, rpos, None, tv, batch, edges, 64, Hh.DIST_MAX, 1.0, Wk, Wax[0], Wax[1], Wax[2], fr[0], fr[1], fr[2],
        64, 4.0, 0, 1.0, 1.0, rv, CUT)
    grads = torch.autograd.grad([z, psi], [a, Wk] + Wax, [g(gz), g(gpsi)])
    return z.detach(), psi.detach(), [f.detach() for f in fr], [x.detach() for x in grads]


def test_large_cell_stress_case_at_full_size():
    P = _large_cell_problem()
    assert len(P.sizes) == 32 and min(P.sizes) >= 40 and max(P.sizes) <= 200 and P.E > 300_000
    gen = torch.Generator().manual_seed(43)
    gz1 = torch.randn(P.E, Hh.H, generator=gen)
    gpsi1 = torch.randn(P.E, Hh.H, Hh.DH, generator=gen)
    gz2 = torch.randn(P.E, Hh.H, generator=gen)
    gpsi2 = torch.randn(P.E, Hh.H, Hh.DH, generator=gen)
    z, psi, fr, gr1 = _layer(P, gz1, gpsi1)
    for t in [z, psi] + fr + gr1:
        assert torch.isfinite(t).all()
    # frames are orthonormal and right-handed
    det = torch.linalg.det(torch.stack(fr, dim=-2).double())
    assert (det - 1).abs().max() < 1e-4

    # the backward pass is linear in the upstream gradients
    _, _, _, gr2 = _layer(P, gz2, gpsi2)
    _, _, _, gr12 = _layer(P, gz1 + gz2, gpsi1 + gpsi2)
    for x1, x2, x12 in zip(gr1, gr2, gr12):
        assert Hh.rel_err(x1 + x2, x12) < 2e-5

    # the smallest crystal alone: identical outputs and input gradient (its items do not see the rest of the batch)
    b = min(range(32), key=lambda i: P.sizes[i])
    S = _slice_crystal(P, b)
    zs, psis, frs, grs = _layer(S, gz1[S.sl_e], gpsi1[S.sl_e])
    assert torch.equal(zs, z[S.sl_e]) and torch.equal(psis, psi[S.sl_e])
    for fa, fb in zip(frs, fr):
        assert torch.equal(fa, fb[S.sl_a])
    assert Hh.rel_err(grs[0], gr1[0][S.sl_a]) < 1e-6

    # ... and against the scalar port of the reference kernels with the frames the search chose
    p = CO.make_params(cutoff_radius=CUT)
    frames64 = [f.cpu().double() for f in frs]
    zc, psic, _ = CO.pe_forward(p, S.a, S.rpos, S.tvecs, S.rvlen, S.batch, S.edges, S.W_k[0], S.W_ax, frames64, "f64")
    assert Hh.rel_err(zs, zc) < 2e-5
    assert Hh.rel_err(psis, psic) < 5e-5
    f1c, f2c = CO.frame_axes(p, S.q, S.k, S.a, S.rpos, S.tvecs, S.rvlen, S.batch, S.edges, "f64")[:2]
    fo = TO.orthonormal_frame(torch.as_tensor(f1c).double(), torch.as_tensor(f2c).double())
    agree = ((frames64[0] - fo[0]).abs().amax(-1) < 1e-4) & ((frames64[1] - fo[1]).abs().amax(-1) < 1e-4)
    assert agree.double().mean() > 0.98      # float32 near-ties between candidates aside

    # rotation of every crystal: z and psi unchanged when the frames rotate along
    gq = torch.Generator().manual_seed(5)
    Q, _ = torch.linalg.qr(torch.randn(3, 3, generator=gq, dtype=torch.float64))
    if torch.det(Q) < 0:
        Q[:, 0] = -Q[:, 0]
    import crystalframer_amd as cf
    fr_rot = [g(f.cpu().double() @ Q.T) for f in fr]
    z2, psi2 = cf.RealEncodingWithFramedProjFuncCUDA.apply(
        g(P.a), g(P.rpos @ Q.T), None, g(P.tvecs @ Q.T), P.batch.to(dev()), P.edges.to(dev()).contiguous(), 64,
        Hh.DIST_MAX, 1.0, g(P.W_k), g(P.W_ax[0]), g(P.W_ax[1]), g(P.W_ax[2]), fr_rot[0], fr_rot[1], fr_rot[2],
        64, 4.0, 0, 1.0, 1.0, g(P.rvlen), CUT)
    assert Hh.rel_err(z2, z) < 2e-5
    assert Hh.rel_err(psi2, psi) < 1e-4


@pytest.mark.parametrize("angle_bins", [64, 0])
def test_inference_batch_of_4096_small_crystals(angle_bins):
    from crystalframer_amd import latticeformer, params, synthetic
    mp = params.ModelParams(num_layers=4, value_pe_angle_real=angle_bins, symm_break_noise=0.0)
    torch.manual_seed(3)
    model = latticeformer.Latticeformer(mp).to(dev())
    cb = synthetic.make_config("C5", seed=123)
    assert cb.num_crystals == 4096
    sizes = cb.sizes.tolist()
    # one training-mode pass on a few crystals fixes the normalisation of alpha, as the first training step does;
    # without it an evaluation pass normalises by the statistics of its own batch
    model.train()
    model(_sub_batch(cb, sizes, range(64)).to(dev()))
    model.eval()
    with torch.no_grad():
        out = model(cb.to(dev()))
        assert out.shape == (4096, 1) and torch.isfinite(out).all()
        # a crystal's output does not depend on the rest of the batch
        first = model(_sub_batch(cb, sizes, range(48)).to(dev()))
        assert Hh.rel_err(first, out[:48]) < 2e-5
        # reordering the crystals reorders the outputs
        order = list(range(4095, -1, -1))
        rev = model(_sub_batch(cb, sizes, order).to(dev()))
        assert Hh.rel_err(rev.flip(0), out) < 2e-5
    assert float(out.std()) > 0


def _sub_batch(cb, sizes, which):
    """The crystals `which` (in that order) of a batch as a batch of their own."""
    from crystalframer_amd.synthetic import CrystalBatch
    starts = [0]
    for s in sizes:
        starts.append(starts[-1] + s)
    which = list(which)
    idx = torch.cat([torch.arange(starts[b], starts[b + 1]) for b in which])
    new_sizes = torch.tensor([sizes[b] for b in which], dtype=cb.sizes.dtype)
    batch = torch.repeat_interleave(torch.arange(len(which)), new_sizes)
    return CrystalBatch(cb.x[idx], cb.pos[idx], batch, cb.trans_vec[torch.tensor(which)], new_sizes)
