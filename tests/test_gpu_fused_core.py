"""The fused attention core (cfh_fused_core_forward / backward through PeriodicAttentionCoreHIP) against the
float64 oracle composition  TO.framed_pe -> TO.softmax_attention  (autograd for every gradient), and against the
two-step operators of the library.  The fused core sums the same translation sets and uses the same distance
windows as the two-step path; its angle encoding is the FULL Gaussian basis (a 5-term series around the nearest
bin), so the oracle runs with windows = (9, None): 9-bin distance window (KernelManager.CORE_WINDOW_MODE = 0 in
this file; the default is the 11-bin window), untruncated angle basis.

Tolerances (relative to the largest magnitude of the tensor): 2e-5 forward, 1e-4 gradients."""
import math

import pytest
import torch

import helpers as Hh
from oracle import torch_oracle as TO

pytestmark = pytest.mark.gpu

CUT = -3.5


@pytest.fixture(autouse=True)
def _defaults():
    import crystalframer_amd as cf
    KM = cf.KernelManager
    names = ("SYMM_BREAK_NOISE", "PRUNE_LOG2", "WINDOW_MODE", "CORE_WINDOW_MODE", "GRAD_COEF_QUIRK", "LATTICE_RANGE",
             "MINIMUM_RANGE", "SAVE_HISTOGRAMS", "SECOND_STREAM", "NOISE_SEED", "NOISE_SEED_DEVICE")
    saved = {n: getattr(KM, n) for n in names}
    KM.SYMM_BREAK_NOISE, KM.PRUNE_LOG2, KM.WINDOW_MODE, KM.GRAD_COEF_QUIRK = 0.0, 24.0, 0, False
    KM.CORE_WINDOW_MODE = 0        # 9-bin distance window unless a test says otherwise (oracle: windows=(9, None))
    KM.LATTICE_RANGE, KM.MINIMUM_RANGE = 2, 2
    yield
    for n, v in saved.items():
        setattr(KM, n, v)


def dev():
    return torch.device("cuda:0")


def g(t):
    return None if t is None else t.to(dtype=torch.float32, device=dev())


def run_core(P, *, A=64, cos_abs=0, cd=1.0, ca=1.0, cutoff=CUT, frames="given", need_grad=True):
    from crystalframer_amd import cuda_funcs as F
    leaves = dict(q=g(P.q), k=g(P.k), v=g(P.v), a=g(P.a), Wk=g(P.W_k))
    if A > 0:
        for n in range(3):
            leaves["W%d" % (n + 1)] = g(P.W_ax[n])
    for t in leaves.values():
        t.requires_grad_(need_grad)
    Wax = [leaves.get("W%d" % n) for n in (1, 2, 3)]
    fr = None
    if A > 0 and frames == "given":
        fr = torch.stack([g(f) for f in P.frames], 0)
    extra = (g(P.rvlen), cutoff) if cutoff is not None else (None, None)
    out, fr_out = F.PeriodicAttentionCoreHIP.apply(
        leaves["q"], leaves["k"], leaves["v"], leaves["a"], g(P.rpos), g(P.tvecs), P.batch.to(dev()), P.edges.to(dev()),
        64, Hh.DIST_MAX, 1.0, leaves["Wk"], Wax[0], Wax[1], Wax[2], A, 4.0, cos_abs, cd, ca, extra[0], extra[1], fr)
    return out, fr_out, leaves


def oracle_core(P, *, A=64, cos_abs=0, cd=1.0, ca=1.0, cutoff=CUT, frames=None, wl=9):
    leaves = dict(q=P.q.clone(), k=P.k.clone(), v=P.v.clone(), a=P.a.clone(), Wk=P.W_k.clone())
    if A > 0:
        for n in range(3):
            leaves["W%d" % (n + 1)] = P.W_ax[n].clone()
    for t in leaves.values():
        t.requires_grad_(True)
    Wax = [leaves["W%d" % n] for n in (1, 2, 3)] if A > 0 else None
    z, psi = TO.framed_pe(leaves["a"], P.rpos, P.tvecs, P.batch, P.edges, leaves["Wk"], Wax, frames or P.frames, K=64,
                          A=A, cos_abs=cos_abs, c_dist=cd, c_angle=ca, rvlen=P.rvlen, cutoff_radius=cutoff,
                          windows=(wl, None))
    out, prob = TO.softmax_attention(leaves["q"], leaves["k"], leaves["v"], z, psi, P.batch, P.edges)
    return out, leaves


def compare(P, gout, out, leaves, oo, oleaves, ftol=2e-5, gtol=1e-4):
    assert torch.isfinite(out).all()
    assert Hh.rel_err(out, oo) < ftol
    (out * g(gout)).sum().backward()
    (oo * gout).sum().backward()
    for name, t in leaves.items():
        assert t.grad is not None and torch.isfinite(t.grad).all(), name
        ref = oleaves[name].grad
        if float(ref.abs().max()) < 1e-12:        # e.g. the query gradient of a one-pair row: exactly zero
            assert float(t.grad.abs().max()) < 1e-5, name
        else:
            assert Hh.rel_err(t.grad, ref) < gtol, name


def _gout(P, seed=77):
    gen = torch.Generator().manual_seed(seed)
    return torch.randn(P.N, Hh.H, Hh.DH, generator=gen, dtype=torch.float64)


@pytest.mark.parametrize("cos_abs", [0, 1])
@pytest.mark.parametrize("prune", [24.0, 0.0])
def test_fused_core_matches_oracle_composition(cos_abs, prune):
    """prune 24: sorted tables and skipped prefixes; prune 0: every translation of every box is evaluated."""
    import crystalframer_amd as cf
    cf.KernelManager.PRUNE_LOG2 = prune
    P = Hh.make_problem(num_crystals=10, atoms_hi=6, seed=200 + cos_abs)
    cd, ca = 0.75, 1.25
    out, _, leaves = run_core(P, cos_abs=cos_abs, cd=cd, ca=ca)
    oo, oleaves = oracle_core(P, cos_abs=cos_abs, cd=cd, ca=ca)
    compare(P, _gout(P), out, leaves, oo, oleaves)


def test_fused_core_distance_encoding_only():
    P = Hh.make_problem(num_crystals=8, atoms_hi=7, seed=211)
    out, fr, leaves = run_core(P, A=0)
    assert fr is None
    oo, oleaves = oracle_core(P, A=0)
    compare(P, _gout(P), out, leaves, oo, oleaves)


def test_fused_core_fixed_box_and_wide_distance_window():
    import crystalframer_amd as cf
    cf.KernelManager.CORE_WINDOW_MODE = 1
    P = Hh.make_problem(num_crystals=8, atoms_hi=5, seed=213)
    out, _, leaves = run_core(P, cutoff=None)
    oo, oleaves = oracle_core(P, cutoff=None, wl=11)
    compare(P, _gout(P), out, leaves, oo, oleaves)
    # and against the untruncated distance basis: the bar of 1e-4
    leaves2 = {k: v.clone().requires_grad_(True) for k, v in dict(q=P.q, k=P.k, v=P.v, a=P.a, Wk=P.W_k).items()}
    z, psi = TO.framed_pe(leaves2["a"], P.rpos, P.tvecs, P.batch, P.edges, leaves2["Wk"], P.W_ax, P.frames,
                          cutoff_radius=None, windows="full")
    of, _ = TO.softmax_attention(leaves2["q"], leaves2["k"], leaves2["v"], z, psi, P.batch, P.edges)
    assert Hh.rel_err(out, of) < 1e-4


def test_fused_core_small_cells_with_boxes_of_several_chunks():
    """Cells of 1.5-2 angstrom: boxes of more than 512 translations (tables rebuilt chunk by chunk)."""
    P = Hh.make_problem(num_crystals=4, atoms_lo=1, atoms_hi=3, len_lo=1.5, len_hi=2.0, ang_lo=80, ang_hi=100, seed=37)
    R = TO.translation_ranges(P.a, P.rvlen, P.batch, CUT)
    assert int((2 * R + 1).prod(-1).max()) > 512
    out, _, leaves = run_core(P)
    oo, oleaves = oracle_core(P)
    compare(P, _gout(P), out, leaves, oo, oleaves)


@pytest.mark.parametrize("shear", [1, 4])
def test_fused_core_sheared_cells(shear):
    """The same lattices described by sheared cells (second cell vector + shear x the first): boxes that contain
    the usual one, whose nearest image of a pair may lie outside the usual box (mildly for shear 1, far outside
    for shear 4)."""
    P = Hh.make_problem(num_crystals=5, atoms_lo=2, atoms_hi=5, len_lo=2.5, len_hi=4.0, seed=223 + shear)
    P.tvecs = P.tvecs.clone()
    P.tvecs[:, 1] += shear * P.tvecs[:, 0]
    P.tvecs = P.tvecs.float().double()
    P.edges, P.rpos, recip, P.vcell = TO.geometry(P.pos, P.tvecs, P.sizes)
    P.rpos = P.rpos.float().double()
    P.rvlen = torch.norm(recip, 2, dim=-1).float().double()
    R = TO.translation_ranges(P.a, P.rvlen, P.batch, CUT)
    assert int(R.max()) > 2 and int((2 * R + 1).prod(-1).max()) <= 8192
    out, _, leaves = run_core(P)
    oo, oleaves = oracle_core(P)
    compare(P, _gout(P), out, leaves, oo, oleaves)


def test_fused_core_more_records_with_boxes_of_their_own_than_leading_wavefronts():
    """28 crystals of small cells: some 600 records whose box is not the usual one, more than the 256 wavefronts
    that take such records first, so the rest are taken in place.  Frames from the search of the same call (equal to
    those of the box search), out and every gradient against the oracle with those frames."""
    P = Hh.make_problem(num_crystals=28, atoms_lo=2, atoms_hi=4, len_lo=2.2, len_hi=3.0, ang_lo=80, ang_hi=100, seed=229)
    R = TO.translation_ranges(P.a, P.rvlen, P.batch, CUT)
    assert int((R.reshape(-1, 3).max(-1).values > 2).sum()) > 300
    fr, ref = _frames_both_ways(P)
    assert torch.equal(fr, ref)
    out, fr2, leaves = run_core(P, frames="search")
    assert torch.equal(fr2, ref)
    oo, oleaves = oracle_core(P, frames=[f.double().cpu() for f in fr2])
    compare(P, _gout(P), out, leaves, oo, oleaves)


def test_fused_core_mixed_boxes_and_long_rows():
    """Crystals of up to 40 atoms (rows of several groups, the running softmax rescales) with cell sizes that
    mix the usual box with larger ones."""
    P = Hh.make_problem(num_crystals=5, atoms_lo=20, atoms_hi=40, len_lo=2.5, len_hi=9.0, seed=219)
    P.q = P.q * 4.0          # sharper attention: larger changes of the running maximum
    out, _, leaves = run_core(P)
    oo, oleaves = oracle_core(P)
    compare(P, _gout(P), out, leaves, oo, oleaves, gtol=2e-4)


def test_fused_core_with_frame_search_equals_two_step_path():
    """frames=None: the search runs in the same call; its frames are those of ComputeFramesMaximumMethodCUDA
    bit for bit, and out equals the two-step operators with those frames up to the truncation of their angle
    windows (5-sigma windows: 1e-4)."""
    import crystalframer_amd as cf
    cf.KernelManager.WINDOW_MODE = cf.KernelManager.CORE_WINDOW_MODE = 1
    P = Hh.make_problem(num_crystals=12, atoms_hi=6, seed=83)
    out, fr, leaves = run_core(P, frames="search")
    ref_fr = cf.ComputeFramesMaximumMethodCUDA.apply(g(P.q), g(P.k), None, g(P.a), g(P.rpos), None, g(P.tvecs),
                                                     P.batch.to(dev()), P.edges.to(dev()), 64, Hh.DIST_MAX, 1.0,
                                                     g(P.rvlen), CUT)
    assert torch.equal(fr, ref_fr)
    z, psi = cf.RealEncodingWithFramedProjFuncCUDA.apply(
        g(P.a), g(P.rpos), None, g(P.tvecs), P.batch.to(dev()), P.edges.to(dev()), 64, Hh.DIST_MAX, 1.0, g(P.W_k),
        g(P.W_ax[0]), g(P.W_ax[1]), g(P.W_ax[2]), fr[0], fr[1], fr[2], 64, 4.0, 0, 1.0, 1.0, g(P.rvlen), CUT)
    two = cf.FusedDotProductAttentionCUDA.apply(g(P.q), g(P.k), g(P.v), z, psi, P.batch.to(dev()), P.edges.to(dev()))
    assert Hh.rel_err(out, two.double().cpu()) < 1e-4
    oo, oleaves = oracle_core(P, frames=[f.double().cpu() for f in fr], wl=11)
    compare(P, _gout(P), out, leaves, oo, oleaves)


def _frames_both_ways(P, cutoff=CUT):
    """Frames of the fused core's own search (translations sorted by length, bounded prefixes) and of
    ComputeFramesMaximumMethodCUDA (whole boxes, slabs skipped): two searches written independently."""
    import crystalframer_amd as cf
    _, fr, _ = run_core(P, frames="search", need_grad=False, cutoff=cutoff)
    extra = (g(P.rvlen), cutoff) if cutoff is not None else ()
    ref = cf.ComputeFramesMaximumMethodCUDA.apply(g(P.q), g(P.k), None, g(P.a), g(P.rpos), None, g(P.tvecs),
                                                  P.batch.to(dev()), P.edges.to(dev()), 64, Hh.DIST_MAX, 1.0, *extra)
    return fr, ref


@pytest.mark.parametrize("noise", [0.0, 1e-5, 1e-2])
def test_sorted_frame_search_equals_the_box_search_at_batch_256(noise):
    """Both searches take the arg-max of the same scores with the same tie rule and, for a given seed, the same
    noise, so the frames are equal bit for bit -- if the bounded prefixes of the sorted search never lose the winner."""
    import crystalframer_amd as cf
    from crystalframer_amd import synthetic
    KM = cf.KernelManager
    KM.SYMM_BREAK_NOISE, KM.NOISE_SEED, KM.NOISE_SEED_DEVICE = noise, 1234567, None
    P = Hh.problem_from_batch(synthetic.make_config("C2"), seed=9)
    fr, ref = _frames_both_ways(P)
    assert torch.equal(fr, ref)
    n = fr.norm(dim=-1)
    assert float((n - 1).abs().max()) < 1e-5


@pytest.mark.parametrize("noise", [0.0, 1e-5])
def test_sorted_frame_search_mixed_boxes_fixed_box_and_long_rows(noise):
    """Small cells (boxes wider than the table's: whole-box scan in chunks), the fixed box without a cutoff, rows
    of more pairs than are staged at once, one-atom crystals (only self images: exact +-n ties)."""
    import crystalframer_amd as cf
    KM = cf.KernelManager
    KM.SYMM_BREAK_NOISE, KM.NOISE_SEED, KM.NOISE_SEED_DEVICE = noise, 99, None
    P = Hh.make_problem(num_crystals=6, atoms_lo=2, atoms_hi=12, len_lo=2.5, len_hi=7.0, seed=301)
    fr, ref = _frames_both_ways(P)
    assert torch.equal(fr, ref)
    fr, ref = _frames_both_ways(P, cutoff=None)
    assert torch.equal(fr, ref)
    P = Hh.make_problem(num_crystals=1, atoms_lo=300, atoms_hi=300, len_lo=14.0, len_hi=16.0, seed=302)
    fr, ref = _frames_both_ways(P)
    assert torch.equal(fr, ref)
    P = Hh.make_problem(num_crystals=7, atoms_lo=1, atoms_hi=1, seed=303)
    fr, ref = _frames_both_ways(P)
    assert torch.equal(fr, ref)


@pytest.mark.parametrize("noise", [0.0, 1e-5])
def test_sorted_frame_search_on_symmetric_crystals_with_exact_ties(noise):
    """Cubic cells with atoms at special positions (simple cubic, body-centred, face-centred, a 2 x 1 x 1 supercell) and
    the SAME query, key and Gaussian width on every atom: several pairs and several translations reach exactly the
    same best score, so the winner is whatever the tie rule says (lowest pair, then lowest translation in the
    reference's loop order).  The sorted search -- which looks only at the pairs whose nearest valid image can hold
    the maximum -- must keep every tied candidate: its frames equal the box search's bit for bit."""
    import crystalframer_amd as cf
    from oracle import torch_oracle as TO
    KM = cf.KernelManager
    KM.SYMM_BREAK_NOISE, KM.NOISE_SEED, KM.NOISE_SEED_DEVICE = noise, 4321, None
    cells = [
        (4.0, [[0, 0, 0]]),
        (3.5, [[0, 0, 0], [0.5, 0.5, 0.5]]),
        (5.0, [[0, 0, 0], [0.5, 0.5, 0], [0.5, 0, 0.5], [0, 0.5, 0.5]]),
        (4.5, [[0, 0, 0], [0.5, 0, 0], [0.25, 0.5, 0.5], [0.75, 0.5, 0.5]]),
        (6.0, [[0.25, 0.25, 0.25], [0.75, 0.75, 0.25], [0.75, 0.25, 0.75], [0.25, 0.75, 0.75],
               [0.75, 0.75, 0.75], [0.25, 0.25, 0.75], [0.25, 0.75, 0.25], [0.75, 0.25, 0.25]]),
    ]
    P = Hh.make_problem(num_crystals=len(cells), atoms_lo=1, atoms_hi=1, seed=77)
    sizes = [len(f) for _, f in cells]
    P.sizes = sizes
    P.tvecs = torch.stack([torch.eye(3, dtype=torch.float64) * a for a, _ in cells])
    P.pos = torch.cat([torch.tensor(f, dtype=torch.float64) * a for a, f in cells])
    P.batch = torch.repeat_interleave(torch.arange(len(cells)), torch.tensor(sizes))
    P.edges, P.rpos, recip, P.vcell = TO.geometry(P.pos, P.tvecs, P.sizes)
    P.rpos = P.rpos.float().double()
    P.rvlen = torch.norm(recip, 2, dim=-1).float().double()
    P.N, P.E = P.pos.shape[0], P.edges.shape[1]
    gen = torch.Generator().manual_seed(5)
    one = lambda *shape: torch.randn(*shape, generator=gen, dtype=torch.float64).float().double()
    P.q = (one(1, Hh.H, Hh.DH) / 4).expand(P.N, -1, -1).contiguous()
    P.k = one(1, Hh.H, Hh.DH).expand(P.N, -1, -1).contiguous()
    P.v = one(P.N, Hh.H, Hh.DH)
    P.a = TO.gaussian_coefficient(one(1, Hh.H)).float().double().expand(P.N, -1).contiguous()
    fr, ref = _frames_both_ways(P)
    assert torch.equal(fr, ref)
    fr, ref = _frames_both_ways(P, cutoff=None)
    assert torch.equal(fr, ref)
    det = torch.linalg.det(fr.permute(1, 2, 0, 3).double())
    assert float((det - 1).abs().max()) < 1e-4


def test_fused_core_one_atom_crystals_and_empty_batch():
    from crystalframer_amd import cuda_funcs as F
    P = Hh.make_problem(num_crystals=5, atoms_lo=1, atoms_hi=1, seed=41)
    out, _, leaves = run_core(P)
    oo, oleaves = oracle_core(P)
    compare(P, _gout(P), out, leaves, oo, oleaves)
    d = dev()
    Wk = g(P.W_k).requires_grad_(True)
    Wax = [g(w).requires_grad_(True) for w in P.W_ax]
    a = torch.zeros(0, Hh.H, device=d, requires_grad=True)
    e3 = torch.zeros(0, Hh.H, Hh.DH, device=d)
    out, fr = F.PeriodicAttentionCoreHIP.apply(
        e3, e3, e3, a, torch.zeros(0, 3, device=d), torch.zeros(0, 3, 3, device=d),
        torch.zeros(0, dtype=torch.long, device=d), torch.zeros(2, 0, dtype=torch.long, device=d), 64, Hh.DIST_MAX, 1.0,
        Wk, *Wax, 64, 4.0, 0, 1.0, 1.0)
    assert out.shape == (0, Hh.H, Hh.DH) and fr.shape == (3, 0, Hh.H, 3)
    out.sum().backward()
    assert float(Wk.grad.abs().max()) == 0.0 and float(Wax[1].grad.abs().max()) == 0.0


def test_fused_core_at_batch_256_against_oracle_on_first_crystals():
    """The benchmark's batch: the core on all 256 crystals; the upstream gradient is zero outside the first 6
    crystals, so every gradient can be compared with the oracle run on those crystals alone."""
    from crystalframer_amd import synthetic
    P = Hh.problem_from_batch(synthetic.make_config("C2"), seed=9)
    S = Hh.first_crystals(P, 6)
    gout = torch.zeros(P.N, Hh.H, Hh.DH, dtype=torch.float64)
    gout[:S.N] = _gout(S, seed=5)
    out, _, leaves = run_core(P)
    oo, oleaves = oracle_core(S)
    assert torch.isfinite(out).all()
    assert Hh.rel_err(out[:S.N], oo) < 2e-5 and Hh.elem_err(out[:S.N], oo, atol_frac=1e-5) <= 1.0
    (out * g(gout)).sum().backward()
    (oo * gout[:S.N]).sum().backward()
    for name in ("q", "k", "v", "a"):
        assert Hh.rel_err(leaves[name].grad[:S.N], oleaves[name].grad) < 1e-4, name
        assert float(leaves[name].grad[S.N:].abs().max()) == 0.0, name
    for name in ("Wk", "W1", "W2", "W3"):
        assert Hh.rel_err(leaves[name].grad, oleaves[name].grad) < 1e-4, name


def test_fused_core_4096_crystals_equals_the_same_crystals_in_reverse_order():
    """4096 crystals (22 375 atoms, 179 000 items, 700 lists of records taken first): every item's result depends on
    its own crystal alone, so the batch with its crystals in reverse order, where every item has another place in the
    work order and in the lists, must give the same frames, the same rows of out and the same gradients."""
    from crystalframer_amd import synthetic
    cb = synthetic.make_config("C5")
    P = Hh.problem_from_batch(cb, seed=11)
    B = len(P.sizes)
    starts = torch.tensor([0] + P.sizes).cumsum(0)
    perm = torch.cat([torch.arange(int(starts[b]), int(starts[b + 1])) for b in reversed(range(B))])
    Q = Hh.Problem()
    Q.sizes = P.sizes[::-1]
    Q.pos, Q.tvecs = P.pos[perm], P.tvecs.flip(0)
    Q.batch = torch.repeat_interleave(torch.arange(B), torch.tensor(Q.sizes))
    Q.edges, Q.rpos, recip, Q.vcell = TO.geometry(Q.pos, Q.tvecs, Q.sizes)
    Q.rvlen = torch.norm(recip, 2, dim=-1)
    Q.N, Q.E = P.N, P.E
    Q.a, Q.q, Q.k, Q.v = P.a[perm], P.q[perm], P.k[perm], P.v[perm]
    Q.W_k, Q.W_ax, Q.frames = P.W_k, P.W_ax, [f[perm] for f in P.frames]
    gout = _gout(P, seed=13)
    res = []
    for prob, go in ((P, gout), (Q, gout[perm])):
        out, fr, leaves = run_core(prob, frames="search")
        assert torch.isfinite(out).all()
        (out * g(go)).sum().backward()
        res.append((out.detach(), fr, {n: t.grad for n, t in leaves.items()}))
    (o1, f1, g1), (o2, f2, g2) = res
    pd = perm.to(dev())
    assert torch.equal(f2, f1[:, pd])
    assert Hh.rel_err(o2, o1[pd]) < 1e-6
    for name in ("q", "k", "v", "a"):
        assert Hh.rel_err(g2[name], g1[name][pd]) < 1e-6, name
    for name in ("Wk", "W1", "W2", "W3"):
        assert Hh.rel_err(g2[name], g1[name]) < 1e-5, name


def test_workspace_header_survives_a_backward_pass():
    """Status word, statistics and work-queue heads at the head of the shared workspace are not scratch: a forward +
    backward pass (with the weight gradients made at the end of the pass) leaves the term counters meaningful and the
    status word clear."""
    import crystalframer_amd as cf
    from crystalframer_amd import _lib
    KM = cf.KernelManager
    P = Hh.make_problem(num_crystals=12, atoms_hi=6, seed=31)
    _lib.read_stats(dev(), reset=True)
    _lib.read_status(dev(), reset=True)
    saved = KM.COLLECT_STATS
    KM.COLLECT_STATS = True
    try:
        out, _, leaves = run_core(P)
        (out * g(_gout(P))).sum().backward()
        torch.cuda.synchronize()
    finally:
        KM.COLLECT_STATS = saved
    st = _lib.read_stats(dev(), reset=True)
    assert _lib.read_status(dev()) == 0
    pairs = P.E * Hh.H
    assert st["fwd_pairs"] == pairs and st["bwd_pairs"] == pairs
    assert 0 < st["fwd_evaluated"] <= st["fwd_in_box"] <= 343 * 2 * pairs
    assert 0 < st["bwd_evaluated"] <= st["bwd_in_box"] == st["fwd_in_box"]
    for name in ("Wk", "W1", "W2", "W3"):
        assert leaves[name].grad is not None and float(leaves[name].grad.abs().max()) > 0


def test_fused_core_reports_pairs_that_are_not_whole_blocks():
    """A caller of the C ABI that hands over another pair layout than the complete n x n block per crystal (here: the
    neighbours of every atom in descending order, declared complete to get past the Python check): the call sets bit 2
    of the workspace's status word, reads inside the arrays and returns finite numbers; with the right layout the bit
    stays clear."""
    from crystalframer_amd import _lib, cuda_funcs as F
    P = Hh.make_problem(num_crystals=6, atoms_lo=2, atoms_hi=5, seed=47)
    _lib.read_status(dev(), reset=True)
    out, _, _ = run_core(P, need_grad=False)
    torch.cuda.synchronize()
    assert _lib.read_status(dev(), reset=True) & 2 == 0
    # reverse the neighbours within every row
    e_dev = P.edges.to(dev())
    rows = torch.bincount(P.edges[0], minlength=P.N)
    start = torch.cumsum(rows, 0) - rows
    pos_in_row = torch.arange(P.E) - start[P.edges[0]]
    perm = start[P.edges[0]] + rows[P.edges[0]] - 1 - pos_in_row
    Q = Hh.Problem()
    Q.__dict__.update(P.__dict__)
    Q.edges, Q.rpos = P.edges[:, perm].contiguous(), P.rpos[perm].contiguous()
    edges_dev = Q.edges.to(dev())
    F.declare_complete_blocks(edges_dev)
    leaves = [g(t) for t in (Q.q, Q.k, Q.v, Q.a)]
    out2, _ = F.PeriodicAttentionCoreHIP.apply(
        *leaves, g(Q.rpos), g(Q.tvecs), Q.batch.to(dev()), edges_dev, 64, Hh.DIST_MAX, 1.0, g(Q.W_k), g(Q.W_ax[0]),
        g(Q.W_ax[1]), g(Q.W_ax[2]), 64, 4.0, 0, 1.0, 1.0, g(Q.rvlen), CUT, torch.stack([g(f) for f in Q.frames], 0))
    torch.cuda.synchronize()
    assert _lib.read_status(dev(), reset=True) & 2 == 2
    assert torch.isfinite(out2).all()
