"""Pins the CPU oracles to facts that do not come from the oracles themselves: closed forms,
textbook identities, brute-force loops on tiny cells, symmetry properties, and agreement between the
two independently written oracles (math-level PyTorch with autograd vs kernel-text-level C with
hand-derived gradients).  Runs on the CPU only."""
import itertools
import math

import numpy as np
import pytest
import torch

import helpers as Hh
from oracle import c_oracle as CO
from oracle import torch_oracle as TO

F64 = torch.float64


@pytest.fixture(autouse=True)
def _float64_default():
    """These tests build their small tensors in float64; restore the default for other modules."""
    old = torch.get_default_dtype()
    torch.set_default_dtype(torch.float64)
    yield
    torch.set_default_dtype(old)


def _one_crystal(lattice, frac):
    tv = torch.tensor(lattice, dtype=F64).reshape(1, 3, 3)
    pos = torch.tensor(frac, dtype=F64) @ tv[0]
    n = pos.shape[0]
    batch = torch.zeros(n, dtype=torch.long)
    edges, rpos, recip, vcell = TO.geometry(pos, tv, [n])
    return tv, pos, batch, edges, rpos, recip, vcell


# ------------------------------------------------------------------------------------------------
# translation-set rule: known answers worked out by hand for a cubic cell
# ------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("L,expect", [(3.0, 2), (2.4, 3), (1.6, 4), (10.0, 2)])
def test_translation_range_known_answers(L, expect):
    # sigma = 1.4  ->  a = -0.5/1.96; cutoff = 3.5*1.4 + 0.01 = 4.91; |b| = 2 pi / L; R = ceil(4.91/L), min 2
    a = torch.full((1, 1), -0.5 / 1.96)
    rvlen = torch.full((1, 3), 2 * math.pi / L)
    R = TO.translation_ranges(a, rvlen, torch.zeros(1, dtype=torch.long), -3.5, 2, 2)
    assert R.tolist() == [[[expect] * 3]]
    assert max(2, math.ceil(4.91 / L)) == expect


def test_translation_range_fixed_grid():
    a = torch.full((2, 3), -0.3)
    R = TO.translation_ranges(a, None, torch.zeros(2, dtype=torch.long), None, lattice_range=2)
    assert (R == 2).all()
    R = TO.translation_ranges(a, torch.ones(1, 3), torch.zeros(2, dtype=torch.long), 0.0, lattice_range=3)
    assert (R == 3).all()


# ------------------------------------------------------------------------------------------------
# z: textbook identities
# ------------------------------------------------------------------------------------------------
def test_z_poisson_identity():
    """sum_n exp(-g|r+nL|^2) = (1/V)(pi/g)^{3/2} sum_G exp(-G^2/4g) cos(G.r)  (Poisson summation)."""
    lattice = [[4.1, 0.0, 0.0], [1.2, 3.7, 0.0], [-0.8, 0.9, 4.4]]
    tv, pos, batch, edges, rpos, recip, vcell = _one_crystal(lattice, [[0.1, 0.2, 0.3], [0.55, 0.8, 0.15]])
    a = torch.tensor([[-0.21, -0.33], [-0.27, -0.4]])
    z = TO.lattice_logsumexp(a, rpos, tv, batch, edges, cutoff_radius=None, lattice_range=9)
    m = torch.tensor(list(itertools.product(range(-8, 9), repeat=3)), dtype=F64)
    G = m @ recip[0]                                   # reciprocal lattice vectors
    G2 = (G * G).sum(-1)
    for e in range(edges.shape[1]):
        i = int(edges[0, e])
        for h in range(2):
            g = -float(a[i, h])
            s = (torch.exp(-G2 / (4 * g)) * torch.cos(G @ rpos[e])).sum()
            ref = math.log(float(s) * (math.pi / g) ** 1.5 / abs(float(vcell[0])))
            assert abs(float(z[e, h]) - ref) < 1e-10


def test_z_orthorhombic_factorisation():
    lattice = [[3.3, 0, 0], [0, 4.7, 0], [0, 0, 5.9]]
    tv, pos, batch, edges, rpos, *_ = _one_crystal(lattice, [[0.2, 0.4, 0.9], [0.7, 0.1, 0.35], [0.5, 0.5, 0.5]])
    a = -0.1 - 0.4 * torch.rand(3, 4, generator=torch.Generator().manual_seed(1))
    R = 3
    z = TO.lattice_logsumexp(a, rpos, tv, batch, edges, cutoff_radius=None, lattice_range=R)
    n = torch.arange(-R, R + 1, dtype=F64)
    for e in range(edges.shape[1]):
        i = int(edges[0, e])
        for h in range(4):
            ref = sum(math.log(float(torch.exp(a[i, h] * (rpos[e, d] + n * lattice[d][d]) ** 2).sum())) for d in range(3))
            assert abs(float(z[e, h]) - ref) < 1e-11


def test_z_lattice_shift_and_basis_change_invariance():
    P = Hh.make_problem(num_crystals=3, atoms_hi=3, seed=5)
    kw = dict(cutoff_radius=None, lattice_range=7)
    z0 = TO.lattice_logsumexp(P.a, P.rpos, P.tvecs, P.batch, P.edges, **kw)
    b = P.batch[P.edges[0]]
    shifted = P.rpos + P.tvecs[b, 0] - 2 * P.tvecs[b, 2]              # add lattice vectors to pos[j]
    assert (TO.lattice_logsumexp(P.a, shifted, P.tvecs, P.batch, P.edges, **kw) - z0).abs().max() < 1e-9
    U = torch.tensor([[1., 1, 0], [0, 1, 0], [0, -1, 1]])             # unimodular change of basis
    assert (TO.lattice_logsumexp(P.a, P.rpos, U @ P.tvecs, P.batch, P.edges, **kw) - z0).abs().max() < 1e-9


def test_sharp_gaussian_limit():
    """a -> -inf: z -> a*d2min and psi -> W.b(d_min)."""
    P = Hh.make_problem(num_crystals=2, atoms_lo=2, atoms_hi=3, seed=2, len_lo=5.0, len_hi=7.0)
    a = torch.full_like(P.a, -60.0)
    z, psi, parts = TO.framed_pe(a, P.rpos, P.tvecs, P.batch, P.edges, P.W_k, None, None, A=0,
                                 cutoff_radius=None, lattice_range=2, windows="full", return_parts=True)
    offdiag = P.edges[0] != P.edges[1]
    d2min = parts["d2min"]
    assert ((z - a[P.edges[0]] * d2min)[offdiag].abs().max()) < 1e-6
    d = d2min.sqrt()
    k = torch.arange(1, 65, dtype=F64) * (14.0 / 64)
    basis = torch.exp(-((k - d[..., None]) / (14.0 / 64)) ** 2 / 2)
    ref = torch.einsum("hck,ehk->ehc", P.W_k[0], basis)
    assert (psi - ref)[offdiag].abs().max() < 1e-6


# ------------------------------------------------------------------------------------------------
# value encodings: brute force with the textbook Gaussian form, and a closed-form cell
# ------------------------------------------------------------------------------------------------
def test_value_pe_brute_force_full_basis():
    lattice = [[3.4, 0.2, 0.0], [0.5, 3.9, 0.1], [0.3, -0.4, 4.2]]
    tv, pos, batch, edges, rpos, *_ = _one_crystal(lattice, [[0.1, 0.2, 0.3], [0.6, 0.7, 0.2]])
    g = torch.Generator().manual_seed(7)
    Hn, Dh, K, A = 2, 3, 64, 64
    a = -0.2 - 0.3 * torch.rand(2, Hn, generator=g)
    W = torch.randn(1, Hn, Dh, K, generator=g)
    Wa = [torch.randn(1, Hn, Dh, A, generator=g) for _ in range(3)]
    fr = [torch.nn.functional.normalize(torch.randn(2, Hn, 3, generator=g), dim=-1) for _ in range(3)]
    z, psi = TO.framed_pe(a, rpos, tv, batch, edges, W, Wa, fr, cutoff_radius=None, lattice_range=2,
                          windows="full", c_dist=0.7, c_angle=1.3)
    sig_d, sig_a = 14.0 / 64, float(np.float32(2 * 4.0 / 63))   # the reference rounds sigma_angle to float32
    for e in range(edges.shape[1]):
        i = int(edges[0, e])
        for h in range(Hn):
            S = 0.0
            hd = np.zeros(K)
            ha = np.zeros((3, A))
            for n1, n2, n3 in itertools.product(range(-2, 3), repeat=3):
                dv = rpos[e] + n1 * tv[0, 0] + n2 * tv[0, 1] + n3 * tv[0, 2]
                d2 = float(dv @ dv)
                w = math.exp(float(a[i, h]) * d2)
                S += w
                d = math.sqrt(d2)
                for kk in range(K):
                    hd[kk] += w * math.exp(-((kk + 1) * 14.0 / 64 - d) ** 2 / (2 * sig_d ** 2))
                if d2 > 1e-5:
                    for ax in range(3):
                        c = float(dv @ fr[ax][i, h]) / d
                        for m in range(A):
                            ha[ax, m] += w * math.exp(-((-1 + 2 * m / 63) - c) ** 2 / (2 * sig_a ** 2))
            assert abs(float(z[e, h]) - math.log(S)) < 1e-10
            ref = 0.7 * (W[0, h].numpy() @ hd) / S
            for ax in range(3):
                ref = ref + 1.3 * (Wa[ax][0, h].numpy() @ ha[ax]) / S
            assert np.abs(psi[e, h].numpy() - ref).max() < 1e-10


def test_angle_pe_one_atom_cubic_closed_form():
    """One atom, cubic cell, frame = cell axes, sharp Gaussian: besides the self image only the six
    nearest images matter and their cosines are exactly 0 or +-1."""
    L = 4.0
    tv, pos, batch, edges, rpos, *_ = _one_crystal([[L, 0, 0], [0, L, 0], [0, 0, L]], [[0.0, 0.0, 0.0]])
    a = torch.tensor([[-1.5]])
    eye = torch.eye(3)
    fr = [eye[d].reshape(1, 1, 3) for d in range(3)]
    W = torch.zeros(1, 1, 1, 64)
    Wa = [torch.zeros(1, 1, 1, 64) for _ in range(3)]
    _, _, parts = TO.framed_pe(a, rpos, tv, batch, edges, W, Wa, fr, cutoff_radius=None, lattice_range=2,
                               windows="full", return_parts=True)
    w1 = math.exp(-1.5 * L * L)
    S = 1 + 6 * w1                                         # next shell: exp(-1.5*2*L^2) ~ 1e-21
    sig = float(np.float32(8.0 / 63))
    mu = -1 + 2 * torch.arange(64, dtype=F64) / 63
    gauss = lambda c: torch.exp(-(mu - c) ** 2 / (2 * sig * sig))
    ref = w1 * (gauss(1.0) + gauss(-1.0) + 4 * gauss(0.0)) / S
    for ax in range(3):
        assert (parts["shat_ang"][ax, 0, 0] - ref).abs().max() < 1e-15


def test_reference_window_drops_only_small_tails():
    """The kernels' 9/33-bin truncation differs from the full basis by at most exp(-8) per term."""
    P = Hh.make_problem(num_crystals=3, atoms_hi=3, seed=11)
    kw = dict(rvlen=P.rvlen, cutoff_radius=-3.5, return_parts=True)
    _, _, full = TO.framed_pe(P.a, P.rpos, P.tvecs, P.batch, P.edges, P.W_k, P.W_ax, P.frames, windows="full", **kw)
    _, _, win = TO.framed_pe(P.a, P.rpos, P.tvecs, P.batch, P.edges, P.W_k, P.W_ax, P.frames, windows="reference", **kw)
    for key in ("shat_len", "shat_ang"):
        diff = full[key] - win[key]
        assert diff.min() >= -1e-15                       # truncation only removes mass
        assert diff.max() <= math.exp(-8.0) * 1.0001      # each dropped bin is beyond 4 sigma
        assert diff.max() > 1e-6                          # and the truncation is really there


# ------------------------------------------------------------------------------------------------
# frames: brute force, orthonormality, SE(3) equivariance
# ------------------------------------------------------------------------------------------------
def _random_rotation(seed):
    g = torch.Generator().manual_seed(seed)
    Q, _ = torch.linalg.qr(torch.randn(3, 3, generator=g))
    if torch.det(Q) < 0:
        Q[:, 0] = -Q[:, 0]
    return Q


def test_frames_brute_force_and_orthonormal():
    P = Hh.make_problem(num_crystals=3, atoms_hi=3, seed=21)
    f1, f2m = TO.frame_axes_max(P.q, P.k, P.a, P.rpos, P.tvecs, P.batch, P.edges, rvlen=P.rvlen, cutoff_radius=-3.5)
    R = TO.translation_ranges(P.a, P.rvlen, P.batch, -3.5)
    # brute force over every (j, n): plain Python loops
    for i in range(P.N):
        b = int(P.batch[i])
        es = [e for e in range(P.E) if int(P.edges[0, e]) == i]
        for h in range(Hh.H):
            best1, best2 = (-1e300, None), (-1e300, None)
            r1, r2, r3 = R[i, h].tolist()
            # first axis: nearest nonzero image per neighbour, then best neighbour
            for e in es:
                j = int(P.edges[1, e])
                qk = float(P.q[i, h] @ P.k[j, h])
                dmin, vmin = 1e300, None
                for n in itertools.product(range(-r1, r1 + 1), range(-r2, r2 + 1), range(-r3, r3 + 1)):
                    dv = P.rpos[e] + n[0] * P.tvecs[b, 0] + n[1] * P.tvecs[b, 1] + n[2] * P.tvecs[b, 2]
                    d2 = float(dv @ dv)
                    if d2 > 1e-5 and d2 < dmin:
                        dmin, vmin = d2, dv
                s = qk + float(P.a[i, h]) * dmin
                if s > best1[0]:
                    best1 = (s, vmin / vmin.norm())
            assert (best1[1] - f1[i, h]).abs().max() < 1e-12
            for e in es:
                j = int(P.edges[1, e])
                qk = float(P.q[i, h] @ P.k[j, h])
                for n in itertools.product(range(-r1, r1 + 1), range(-r2, r2 + 1), range(-r3, r3 + 1)):
                    dv = P.rpos[e] + n[0] * P.tvecs[b, 0] + n[1] * P.tvecs[b, 1] + n[2] * P.tvecs[b, 2]
                    d2 = float(dv @ dv)
                    if d2 <= 1e-5:
                        continue
                    u = dv / math.sqrt(d2)
                    c = abs(float(u @ f1[i, h]))
                    if c >= 0.9999:
                        continue
                    s = qk + float(P.a[i, h]) * d2 + math.log(max(1 - c, 1e-5))
                    if s > best2[0] + 1e-12:              # first in loop order wins exact ties
                        best2 = (s, u)
            assert (best2[1] - f2m[i, h]).abs().max() < 1e-12
    f1, f2, f3 = TO.orthonormal_frame(f1, f2m)
    M = torch.stack([f1, f2, f3], dim=-2)
    assert (M @ M.transpose(-1, -2) - torch.eye(3)).abs().max() < 1e-12
    assert (torch.linalg.det(M) - 1).abs().max() < 1e-12


def test_se3_equivariance_of_frames_and_invariance_of_outputs():
    P = Hh.make_problem(num_crystals=3, atoms_hi=4, seed=31)
    Q = _random_rotation(3)
    kw = dict(rvlen=P.rvlen, cutoff_radius=-3.5)
    f1, f2m = TO.frame_axes_max(P.q, P.k, P.a, P.rpos, P.tvecs, P.batch, P.edges, **kw)
    fr = TO.orthonormal_frame(f1, f2m)
    z, psi = TO.framed_pe(P.a, P.rpos, P.tvecs, P.batch, P.edges, P.W_k, P.W_ax, fr, windows="full", **kw)
    rpos_r, tv_r = P.rpos @ Q.T, P.tvecs @ Q.T
    g1, g2m = TO.frame_axes_max(P.q, P.k, P.a, rpos_r, tv_r, P.batch, P.edges, **kw)
    gr = TO.orthonormal_frame(g1, g2m)
    for f, g in zip(fr, gr):
        assert (f @ Q.T - g).abs().max() < 1e-9
    z2, psi2 = TO.framed_pe(P.a, rpos_r, tv_r, P.batch, P.edges, P.W_k, P.W_ax, gr, windows="full", **kw)
    assert (z - z2).abs().max() < 1e-9
    assert (psi - psi2).abs().max() < 1e-9


# ------------------------------------------------------------------------------------------------
# the two oracles against each other (forward, hand-derived backward vs autograd, frames)
# ------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("windows", ["reference", "full"])
@pytest.mark.parametrize("cos_abs", [0, 1])
def test_c_oracle_matches_torch_oracle_forward_backward(windows, cos_abs):
    P = Hh.make_problem(num_crystals=4, atoms_hi=4, seed=41 + cos_abs)
    cd, ca = 0.75, 1.25          # float32-representable: the C oracle keeps its scalars in float
    a = P.a.clone().requires_grad_(True)
    Wk = P.W_k.clone().requires_grad_(True)
    Wax = [w.clone().requires_grad_(True) for w in P.W_ax]
    z, psi = TO.framed_pe(a, P.rpos, P.tvecs, P.batch, P.edges, Wk, Wax, P.frames, rvlen=P.rvlen,
                          cutoff_radius=-3.5, windows=windows, cos_abs=cos_abs, c_dist=cd, c_angle=ca)
    ((z * P.gz).sum() + (psi * P.gpsi).sum()).backward()
    p = CO.make_params(cos_abs=cos_abs, dist_coef=cd, angle_coef=ca, cutoff_radius=-3.5, windows=windows)
    zc, psic, _ = CO.pe_forward(p, P.a, P.rpos, P.tvecs, P.rvlen, P.batch, P.edges, P.W_k[0], P.W_ax, P.frames, "f64")
    assert Hh.rel_err(zc, z.detach()) < 1e-12
    assert Hh.rel_err(psic, psi.detach()) < 1e-11
    ga, gWd, gWa = CO.pe_backward(p, P.a, P.rpos, P.tvecs, P.rvlen, P.batch, P.edges, P.W_k[0], P.W_ax, P.frames,
                                  zc, P.gz, P.gpsi, "f64")
    assert Hh.rel_err(ga, a.grad) < 1e-10
    assert Hh.rel_err(gWd, Wk.grad[0]) < 1e-10
    for ax in range(3):
        assert Hh.rel_err(gWa[ax], Wax[ax].grad[0]) < 1e-10
    # float32 arithmetic of the reference stays within 1e-4 of the float64 result
    zf, psif, _ = CO.pe_forward(p, P.a, P.rpos, P.tvecs, P.rvlen, P.batch, P.edges, P.W_k[0], P.W_ax, P.frames, "f32")
    assert Hh.rel_err(zf, z.detach()) < 1e-5
    assert Hh.rel_err(psif, psi.detach()) < 1e-4


def test_c_oracle_z_only_and_distance_only_gradients():
    P = Hh.make_problem(num_crystals=3, atoms_hi=4, seed=43)
    a = P.a.clone().requires_grad_(True)
    z = TO.lattice_logsumexp(a, P.rpos, P.tvecs, P.batch, P.edges, rvlen=P.rvlen, cutoff_radius=-3.5)
    (z * P.gz).sum().backward()
    p = CO.make_params(K=0, A=0, cutoff_radius=-3.5)
    zc, _, _ = CO.pe_forward(p, P.a, P.rpos, P.tvecs, P.rvlen, P.batch, P.edges, None, None, None, "f64")
    ga, _, _ = CO.pe_backward(p, P.a, P.rpos, P.tvecs, P.rvlen, P.batch, P.edges, None, None, None, zc, P.gz, None, "f64")
    assert Hh.rel_err(zc, z.detach()) < 1e-12
    assert Hh.rel_err(ga, a.grad) < 1e-11
    # the closed form of dz/da: sum_n p_n d_n^2 (commented restatement in
    # models/cuda_funcs/real_space_enc.py:143-161 of the reference)
    a2 = P.a.clone().requires_grad_(True)
    Wk = P.W_k.clone().requires_grad_(True)
    z, psi = TO.framed_pe(a2, P.rpos, P.tvecs, P.batch, P.edges, Wk, None, None, A=0, rvlen=P.rvlen, cutoff_radius=-3.5)
    ((z * P.gz).sum() + (psi * P.gpsi).sum()).backward()
    p = CO.make_params(A=0, cutoff_radius=-3.5)
    zc, psic, _ = CO.pe_forward(p, P.a, P.rpos, P.tvecs, P.rvlen, P.batch, P.edges, P.W_k[0], None, None, "f64")
    ga, gWd, _ = CO.pe_backward(p, P.a, P.rpos, P.tvecs, P.rvlen, P.batch, P.edges, P.W_k[0], None, None, zc, P.gz,
                                P.gpsi, "f64")
    assert Hh.rel_err(psic, psi.detach()) < 1e-11
    assert Hh.rel_err(ga, a2.grad) < 1e-10
    assert Hh.rel_err(gWd, Wk.grad[0]) < 1e-10


def test_gradient_coefficient_quirk_is_what_the_reference_text_does():
    """With dist_coef != 1 the reference scales the dz/da part by dist_coef and leaves dW_dist unscaled
    (models/cuda_funcs/real_space_framed_proj.py:183-184); the exact gradient does neither."""
    P = Hh.make_problem(num_crystals=2, atoms_hi=3, seed=47)
    cd = 0.5
    common = (P.a, P.rpos, P.tvecs, P.rvlen, P.batch, P.edges, P.W_k[0], None, None)
    pe = CO.make_params(A=0, dist_coef=cd, cutoff_radius=-3.5)
    pq = CO.make_params(A=0, dist_coef=cd, cutoff_radius=-3.5, grad_coef_quirk=True)
    z, _, _ = CO.pe_forward(pe, *common, "f64")
    zero = torch.zeros_like(P.gpsi)
    ga_e, gW_e, _ = CO.pe_backward(pe, *common, z, P.gz, zero, "f64")
    ga_q, gW_q, _ = CO.pe_backward(pq, *common, z, P.gz, zero, "f64")
    assert Hh.rel_err(ga_q, cd * ga_e) < 1e-12             # only the dz/da part is present here
    ga_e, gW_e, _ = CO.pe_backward(pe, *common, z, torch.zeros_like(P.gz), P.gpsi, "f64")
    ga_q, gW_q, _ = CO.pe_backward(pq, *common, z, torch.zeros_like(P.gz), P.gpsi, "f64")
    assert Hh.rel_err(ga_q, ga_e) < 1e-12
    assert Hh.rel_err(gW_q * cd, gW_e) < 1e-12


def test_c_oracle_frames_match_torch_oracle():
    P = Hh.make_problem(num_crystals=5, atoms_hi=4, seed=53)
    f1, f2, gap1, gap2 = TO.frame_axes_max(P.q, P.k, P.a, P.rpos, P.tvecs, P.batch, P.edges, rvlen=P.rvlen,
                                           cutoff_radius=-3.5, return_gaps=True)
    p = CO.make_params(cutoff_radius=-3.5)
    c1, c2 = CO.frame_axes(p, P.q, P.k, P.a, P.rpos, P.tvecs, P.rvlen, P.batch, P.edges, "f64")
    assert (c1 - f1).abs().max() < 1e-12
    assert (c2 - f2).abs().max() < 1e-12
    # float32 search picks the same images wherever the winner is not within rounding of the runner-up
    s1, s2 = CO.frame_axes(p, P.q, P.k, P.a, P.rpos, P.tvecs, P.rvlen, P.batch, P.edges, "f32")
    clear = (gap1 > 1e-4) & (gap2 > 1e-4)
    assert clear.float().mean() > 0.9
    assert (s1.double() - f1)[clear].abs().max() < 1e-5


# ------------------------------------------------------------------------------------------------
# consumer ops
# ------------------------------------------------------------------------------------------------
def test_softmax_attention_oracles_agree_and_match_autograd():
    P = Hh.make_problem(num_crystals=4, atoms_hi=4, seed=61)
    g = torch.Generator().manual_seed(3)
    z = torch.randn(P.E, Hh.H, generator=g)
    psi = torch.randn(P.E, Hh.H, Hh.DH, generator=g)
    gout = torch.randn(P.N, Hh.H, Hh.DH, generator=g)
    leaves = [t.clone().requires_grad_(True) for t in (P.q, P.k, P.v, z, psi)]
    out, prob = TO.softmax_attention(*leaves, P.batch, P.edges)
    # per-crystal dense softmax (torch.softmax) as the textbook reference
    off = 0
    for n in P.sizes:
        sl = slice(off, off + n)
        logits = torch.einsum("ihd,jhd->ijh", P.q[sl], P.k[sl]) + z[P.edges[0] >= off][: n * n].reshape(n, n, Hh.H)
        pr = torch.softmax(logits, dim=1)
        e0 = int(((P.edges[0] < off).sum()))
        vals = P.v[sl][None] + psi[e0:e0 + n * n].reshape(n, n, Hh.H, Hh.DH)
        ref = (pr[..., None] * vals).sum(1)
        assert (ref - out[sl].detach()).abs().max() < 1e-12
        off += n
    (out * gout).sum().backward()
    oc, pc = CO.dpa_forward(P.q, P.k, P.v, z, psi, P.edges, "f64")
    assert Hh.rel_err(oc, out.detach()) < 1e-12
    grads = CO.dpa_backward(P.q, P.k, P.v, psi, P.edges, pc, oc, gout, "f64")
    for gc, leaf in zip(grads, leaves):
        assert Hh.rel_err(gc, leaf.grad) < 1e-11


def test_crystal_mean():
    x = torch.randn(9, 5)
    sizes = [2, 3, 4]
    ref = torch.stack([c.mean(0) for c in torch.split(x, sizes)])
    assert (CO.crystal_mean(x, sizes, "f64") - ref).abs().max() < 1e-14
    batch = torch.repeat_interleave(torch.arange(3), torch.tensor(sizes))
    assert (TO.crystal_mean(x, batch, 3) - ref).abs().max() < 1e-14


# ------------------------------------------------------------------------------------------------
# alpha -> a
# ------------------------------------------------------------------------------------------------
def test_gaussian_coefficient_closed_form_facts():
    """What the formula a = [(1-lb) elu(alpha beta/(1-lb)) + 1] (-1/2 r0^-2) fixes without restating it:
    its value at 0, its limit for alpha -> -inf (the lower bound lb of the positive function), its slope
    for alpha > 0, and that value and slope are continuous at 0."""
    r0, lb, beta = 1.4, 0.5, 0.1
    c2 = -0.5 / (r0 * r0)                                  # -0.25510...
    f = lambda x: float(TO.gaussian_coefficient(torch.tensor([x], dtype=torch.float64), r0, lb, beta))
    assert abs(f(0.0) - c2) < 1e-15
    assert abs(c2 - (-0.25510204081632654)) < 1e-15
    assert abs(f(-1e4) - lb * c2) < 1e-15                  # -> lb (-1/2 r0^-2) = -0.12755...
    assert abs(lb * c2 - (-0.12755102040816327)) < 1e-15
    # linear with slope beta (-1/2 r0^-2) on the positive side
    assert abs((f(7.0) - f(3.0)) / 4.0 - beta * c2) < 1e-15
    assert abs(f(5.0) - (1.0 + beta * 5.0) * c2) < 1e-15
    # C^1 at 0: one-sided difference quotients agree with the slope beta c2
    h = 1e-6
    assert abs((f(h) - f(0.0)) / h - beta * c2) < 1e-9
    assert abs((f(0.0) - f(-h)) / h - beta * c2) < 1e-6
    # monotone: a larger alpha gives a sharper Gaussian (more negative a), always below lb c2
    xs = torch.linspace(-50, 50, 2001, dtype=torch.float64)
    a = TO.gaussian_coefficient(xs, r0, lb, beta)
    assert bool((a[1:] < a[:-1]).all()) and float(a.max()) < lb * c2 + 1e-12
    # other constants: the limit and the slope follow lb and beta
    a2 = TO.gaussian_coefficient(torch.tensor([-1e4, 2.0], dtype=torch.float64), 2.0, 0.25, 0.3)
    assert abs(float(a2[0]) - 0.25 * (-0.125)) < 1e-15 and abs(float(a2[1]) - 1.6 * (-0.125)) < 1e-15


def test_per_pair_weight_sets_reduce_to_the_shared_set_and_select_by_pair_or_atom():
    """W_num = E / N (models/kernels/real_enc_frame_proj_fwd_length.cu:166-173): equal sets give the shared result;
    with distinct sets pair e uses set e (or the set of its query atom): checked by projecting the shared run's
    histograms by hand."""
    P = Hh.make_problem(num_crystals=3, atoms_hi=4, seed=5)
    kw = dict(rvlen=P.rvlen, cutoff_radius=-3.5)
    z, psi, parts = TO.framed_pe(P.a, P.rpos, P.tvecs, P.batch, P.edges, P.W_k, P.W_ax, P.frames, return_parts=True, **kw)
    for num in (P.E, P.N):
        rep = lambda w: w.expand(num, *w.shape[1:]).clone()
        z2, psi2 = TO.framed_pe(P.a, P.rpos, P.tvecs, P.batch, P.edges, rep(P.W_k), [rep(w) for w in P.W_ax], P.frames, **kw)
        assert (z2 - z).abs().max() == 0 and (psi2 - psi).abs().max() < 1e-14
        gen = torch.Generator().manual_seed(num)
        Wk = torch.randn(num, Hh.H, Hh.DH, Hh.K, generator=gen, dtype=torch.float64)
        Wax = [torch.randn(num, Hh.H, Hh.DH, Hh.A, generator=gen, dtype=torch.float64) for _ in range(3)]
        _, psi3 = TO.framed_pe(P.a, P.rpos, P.tvecs, P.batch, P.edges, Wk, Wax, P.frames, **kw)
        rows = torch.arange(P.E) if num == P.E else P.edges[0]
        want = torch.zeros_like(psi3)
        for e in range(P.E):
            for h in range(Hh.H):
                want[e, h] = Wk[rows[e], h] @ parts["shat_len"][e, h]
                for ax in range(3):
                    want[e, h] += Wax[ax][rows[e], h] @ parts["shat_ang"][ax, e, h]
        assert (psi3 - want).abs().max() < 1e-12
