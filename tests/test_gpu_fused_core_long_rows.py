"""The fused attention core (cfh_fused_core_forward / backward through PeriodicAttentionCoreHIP) on rows of MORE
pairs than the 64 logits a wavefront keeps in LDS: crystals of 66-90 atoms, one of 200 atoms, and the large-cell
stress configuration (32 crystals of 40-200 atoms, half a million pairs) at its full size.  On such rows the
kernel parks the logits in the probability array until the row is complete, the running softmax rescales the
item's histogram over dozens of groups of pairs, and the column kernel of the attention backward sums over long
columns.

Oracle: the scalar C port in float64 for z, psi and their backward (the tensor oracle needs minutes and tens of
GB at these sizes), composed with the float64 softmax attention of the tensor oracle, whose autograd gives the
gradients of q, k, v and the upstream gradients (gz, gpsi) of the C port's backward.  The frames are those the
call itself searched.  Windows as the core computes them: the distance window of KernelManager.CORE_WINDOW_MODE,
the angle basis untruncated (C port: angle_range = 0).

Tolerances (relative to the tensor's largest magnitude): forward 2e-5, gradients 1e-4; element-wise bound too."""
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
    names = ("SYMM_BREAK_NOISE", "PRUNE_LOG2", "CORE_WINDOW_MODE", "GRAD_COEF_QUIRK", "LATTICE_RANGE", "MINIMUM_RANGE",
             "NOISE_SEED", "NOISE_SEED_DEVICE")
    saved = {n: getattr(KM, n) for n in names}
    KM.SYMM_BREAK_NOISE, KM.PRUNE_LOG2, KM.GRAD_COEF_QUIRK = 0.0, 24.0, False
    KM.LATTICE_RANGE, KM.MINIMUM_RANGE = 2, 2
    yield
    for n, v in saved.items():
        setattr(KM, n, v)


def dev():
    return torch.device("cuda:0")


def g(t):
    return None if t is None else t.to(dtype=torch.float32, device=dev())


NAMES = ("q", "k", "v", "a", "Wk", "W1", "W2", "W3")


def run_core(P, gout):
    """Forward with the frame search in the call, backward with ``gout``: out, frames, gradients by name."""
    from crystalframer_amd import cuda_funcs as F
    leaves = dict(q=g(P.q), k=g(P.k), v=g(P.v), a=g(P.a), Wk=g(P.W_k), W1=g(P.W_ax[0]), W2=g(P.W_ax[1]),
                  W3=g(P.W_ax[2]))
    for t in leaves.values():
        t.requires_grad_(True)
    out, fr = F.PeriodicAttentionCoreHIP.apply(
        leaves["q"], leaves["k"], leaves["v"], leaves["a"], g(P.rpos), g(P.tvecs), P.batch.to(dev()),
        P.edges.to(dev()).contiguous(), 64, Hh.DIST_MAX, 1.0, leaves["Wk"], leaves["W1"], leaves["W2"], leaves["W3"],
        64, 4.0, 0, 1.0, 1.0, g(P.rvlen), CUT, None)
    grads = torch.autograd.grad(out, [leaves[n] for n in NAMES], g(gout))
    return out.detach(), fr.detach(), dict(zip(NAMES, (x.detach() for x in grads)))


def oracle_core(P, frames, gout, wl):
    """The same composition in float64: C port (z, psi), tensor oracle (softmax over the pairs), autograd for the
    attention, C port for the backward of z and psi."""
    p = CO.make_params(cutoff_radius=CUT, windows=(wl, 0))
    fr64 = [f.double().cpu() for f in frames]
    z, psi, _ = CO.pe_forward(p, P.a, P.rpos, P.tvecs, P.rvlen, P.batch, P.edges, P.W_k[0], P.W_ax, fr64, "f64")
    lv = [t.clone().requires_grad_(True) for t in (P.q, P.k, P.v, z, psi)]
    out, _ = TO.softmax_attention(*lv, P.batch, P.edges)
    (out * gout).sum().backward()
    ga, gWd, gWa = CO.pe_backward(p, P.a, P.rpos, P.tvecs, P.rvlen, P.batch, P.edges, P.W_k[0], P.W_ax, fr64, z,
                                  lv[3].grad, lv[4].grad, "f64")
    grads = dict(q=lv[0].grad, k=lv[1].grad, v=lv[2].grad, a=ga, Wk=gWd[None], W1=gWa[0][None], W2=gWa[1][None],
                 W3=gWa[2][None])
    return out.detach(), grads


def check(out, grads, oo, ogr, ftol=2e-5, gtol=1e-4):
    assert torch.isfinite(out).all()
    assert Hh.rel_err(out, oo) < ftol
    assert Hh.elem_err(out, oo, rtol=1e-4, atol_frac=1e-5) <= 1.0
    for n in NAMES:
        assert torch.isfinite(grads[n]).all(), n
        assert Hh.rel_err(grads[n], ogr[n]) < gtol, n
        assert Hh.elem_err(grads[n], ogr[n], rtol=1e-3, atol_frac=1e-4) <= 1.0, n


def _gout(N, seed):
    return torch.randn(N, Hh.H, Hh.DH, generator=torch.Generator().manual_seed(seed), dtype=torch.float64)


@pytest.mark.parametrize("window_mode,wl", [(0, 9), (1, 11)])
def test_fused_core_rows_of_66_to_90_pairs(window_mode, wl):
    import crystalframer_amd as cf
    cf.KernelManager.CORE_WINDOW_MODE = window_mode
    P = Hh.make_problem(num_crystals=2, atoms_lo=66, atoms_hi=90, len_lo=8.0, len_hi=14.0, seed=301)
    assert min(P.sizes) > 64
    P.q = P.q * 3.0            # sharper attention: the running maximum moves over the groups of a row
    gout = _gout(P.N, 17)
    out, fr, grads = run_core(P, gout)
    oo, ogr = oracle_core(P, fr, gout, wl)
    check(out, grads, oo, ogr)


def test_fused_core_row_of_200_pairs():
    import crystalframer_amd as cf
    cf.KernelManager.CORE_WINDOW_MODE = 0
    P = Hh.make_problem(num_crystals=1, atoms_lo=200, atoms_hi=200, len_lo=14.0, len_hi=18.0, seed=305)
    gout = _gout(P.N, 19)
    out, fr, grads = run_core(P, gout)
    oo, ogr = oracle_core(P, fr, gout, 9)
    check(out, grads, oo, ogr)


def _large_cell_problem():
    from crystalframer_amd import synthetic
    cb = synthetic.make_config("C4", seed=123)
    P = Hh.problem_from_batch(cb, seed=41)
    P.rpos = P.rpos.float().double()
    P.rvlen = P.rvlen.float().double()
    return P


def _slice_crystal(P, b):
    """Atoms, pairs and lattice of crystal b as a problem of its own."""
    a0 = sum(P.sizes[:b])
    e0 = sum(s * s for s in P.sizes[:b])
    n = P.sizes[b]
    S = Hh.Problem()
    S.sl_a, S.sl_e = slice(a0, a0 + n), slice(e0, e0 + n * n)
    S.a, S.q, S.k, S.v = P.a[S.sl_a], P.q[S.sl_a], P.k[S.sl_a], P.v[S.sl_a]
    S.rpos, S.edges = P.rpos[S.sl_e], P.edges[:, S.sl_e] - a0
    S.batch = torch.zeros(n, dtype=torch.long)
    S.tvecs, S.rvlen = P.tvecs[b:b + 1], P.rvlen[b:b + 1]
    S.W_k, S.W_ax = P.W_k, P.W_ax
    S.N, S.E, S.sizes = n, n * n, [n]
    return S


def test_fused_core_large_cell_stress_case_at_full_size():
    """32 crystals of 40-200 atoms through the fused core.  The oracle cannot run the whole batch, so: the smallest
    crystal alone gives the same rows bit for bit (an item sees its own crystal only) and those rows agree with the
    float64 oracle, with an upstream gradient that is zero outside that crystal so that the weight gradients can be
    compared too; the backward pass is linear in the upstream gradient over the whole batch; frames orthonormal."""
    import crystalframer_amd as cf
    cf.KernelManager.CORE_WINDOW_MODE = 0
    P = _large_cell_problem()
    assert len(P.sizes) == 32 and min(P.sizes) >= 40 and max(P.sizes) > 150 and P.E > 300_000
    g1, g2 = _gout(P.N, 43), _gout(P.N, 44)
    out, fr, gr1 = run_core(P, g1)
    assert torch.isfinite(out).all()
    det = torch.linalg.det(fr.permute(1, 2, 0, 3).double())
    assert float((det - 1).abs().max()) < 1e-4

    # linear in the upstream gradient
    _, _, gr2 = run_core(P, g2)
    _, _, gr12 = run_core(P, g1 + g2)
    for n in NAMES:
        assert Hh.rel_err(gr1[n] + gr2[n], gr12[n]) < 2e-5, n

    # the smallest crystal alone: bit-equal rows
    b = min(range(32), key=lambda i: P.sizes[i])
    S = _slice_crystal(P, b)
    outs, frs, grs = run_core(S, g1[S.sl_a])
    assert torch.equal(frs, fr[:, S.sl_a])
    assert torch.equal(outs, out[S.sl_a])
    for n in ("q", "a"):        # sums over the atom's own row: same order of additions
        assert torch.equal(grs[n], gr1[n][S.sl_a]), n
    for n in ("k", "v"):
        assert Hh.rel_err(grs[n], gr1[n][S.sl_a]) < 1e-6, n

    # ... against the oracle, and the whole batch with an upstream gradient confined to that crystal
    oo, ogr = oracle_core(S, frs, g1[S.sl_a], 9)
    check(outs, grs, oo, ogr)
    gm = torch.zeros_like(g1)
    gm[S.sl_a] = g1[S.sl_a]
    _, _, grm = run_core(P, gm)
    for n in ("q", "k", "v", "a"):
        assert Hh.rel_err(grm[n][S.sl_a], ogr[n]) < 1e-4, n
        rest = torch.ones(P.N, dtype=torch.bool)
        rest[S.sl_a] = False
        assert float(grm[n][rest.to(dev())].abs().max()) == 0.0, n
    for n in ("Wk", "W1", "W2", "W3"):
        assert Hh.rel_err(grm[n], ogr[n]) < 1e-4, n

    # the largest crystal against the oracle as well (rows of up to 200 pairs inside the big batch): forward only
    bl = max(range(32), key=lambda i: P.sizes[i])
    L = _slice_crystal(P, bl)
    p = CO.make_params(cutoff_radius=CUT, windows=(9, 0))
    fr64 = [f.double().cpu() for f in fr[:, L.sl_a]]
    z, psi, _ = CO.pe_forward(p, L.a, L.rpos, L.tvecs, L.rvlen, L.batch, L.edges, L.W_k[0], L.W_ax, fr64, "f64")
    ol, _ = TO.softmax_attention(L.q, L.k, L.v, z, psi, L.batch, L.edges)
    assert Hh.rel_err(out[L.sl_a], ol) < 2e-5
    assert Hh.elem_err(out[L.sl_a], ol, rtol=1e-4, atol_frac=1e-5) <= 1.0
