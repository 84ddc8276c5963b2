"""The 16-bin angle basis of the reference's lightweight setting (train_jarvis_time.sh:40-57:
value_pe_angle_real 16, value_pe_angle_wscale 1.0, value_pe_dist_coef 1.5, value_pe_angle_coef 6.0).

With 16 bins the reference's window (ANGLE_RANGE = ceil(8 wscale + 1), models/cuda_funcs/kernel_manager.py:147) leaves
at most 7 bins out, and its kernels then evaluate the WHOLE basis (the windowed branch needs more than 8,
models/kernels/real_enc_frame_proj_fwd_angle.cu:154,168-175), for |cos| as well.  The oracles apply the same rule.

Tolerances (relative to the tensor's largest magnitude): forward 2e-5, gradients 5e-5 (fused core: 1e-4), float32
port of the kernel text 5e-5, model output and parameter gradients 1e-4."""
import pytest
import torch

import helpers as Hh
from oracle import c_oracle as CO
from oracle import cpu_model
from oracle import torch_oracle as TO

pytestmark = pytest.mark.gpu
CUT = -3.5
A16 = 16


@pytest.fixture(autouse=True)
def _defaults():
    import crystalframer_amd as cf
    KM = cf.KernelManager
    names = ("SYMM_BREAK_NOISE", "PRUNE_LOG2", "WINDOW_MODE", "GRAD_COEF_QUIRK", "LATTICE_RANGE", "MINIMUM_RANGE",
             "SAVE_HISTOGRAMS", "SECOND_STREAM")
    saved = {n: getattr(KM, n) for n in names}
    KM.SYMM_BREAK_NOISE, KM.PRUNE_LOG2, KM.WINDOW_MODE, KM.GRAD_COEF_QUIRK = 0.0, 24.0, 0, False
    KM.LATTICE_RANGE, KM.MINIMUM_RANGE = 2, 2
    yield
    for n, v in saved.items():
        setattr(KM, n, v)


def dev():
    return torch.device("cuda:0")


def g(t):
    return None if t is None else t.to(dtype=torch.float32, device=dev())


def _weights16(P, seed=5):
    gen = torch.Generator().manual_seed(seed)
    return [(torch.randn(1, Hh.H, Hh.DH, A16, generator=gen, dtype=torch.float64) * 0.3).float().double() for _ in range(3)]


@pytest.mark.parametrize("cos_abs", [0, 1])
@pytest.mark.parametrize("wscale", [1.0, 4.0])
@pytest.mark.parametrize("save_histograms,window_mode", [(True, 0), (False, 0), (True, 1)])
def test_sixteen_angle_bins_forward_backward(cos_abs, wscale, save_histograms, window_mode):
    import crystalframer_amd as cf
    KM = cf.KernelManager
    KM.SAVE_HISTOGRAMS, KM.WINDOW_MODE = save_histograms, window_mode
    P = Hh.make_problem(num_crystals=10, atoms_hi=6, seed=140 + cos_abs)
    W16 = _weights16(P)
    cd, ca = 1.5, 6.0
    a = g(P.a).requires_grad_(True)
    Wk = g(P.W_k).requires_grad_(True)
    Wax = [g(w).requires_grad_(True) for w in W16]
    fr = [g(f) for f in P.frames]
    z, psi = cf.RealEncodingWithFramedProjFuncCUDA.apply(
        a, g(P.rpos), None, g(P.tvecs), P.batch.to(dev()), P.edges.to(dev()), 64, Hh.DIST_MAX, 1.0, Wk, Wax[0], Wax[1],
        Wax[2], fr[0], fr[1], fr[2], A16, wscale, cos_abs, cd, ca, g(P.rvlen), CUT)
    ao = P.a.clone().requires_grad_(True)
    Wko = P.W_k.clone().requires_grad_(True)
    Waxo = [w.clone().requires_grad_(True) for w in W16]
    # distance window of the library's mode (9 or 11 bins), whole angle basis
    zo, psio = TO.framed_pe(ao, P.rpos, P.tvecs, P.batch, P.edges, Wko, Waxo, P.frames, K=64, A=A16, angle_wscale=wscale,
                            cos_abs=cos_abs, c_dist=cd, c_angle=ca, rvlen=P.rvlen, cutoff_radius=CUT,
                            windows=(9 if window_mode == 0 else 11, None))
    assert Hh.rel_err(z, zo) < 2e-5
    assert Hh.rel_err(psi, psio) < 2e-5 and Hh.elem_err(psi, psio, atol_frac=1e-5) <= 1.0
    ((z * g(P.gz)).sum() + (psi * g(P.gpsi)).sum()).backward()
    ((zo * P.gz).sum() + (psio * P.gpsi).sum()).backward()
    assert Hh.rel_err(a.grad, ao.grad) < 5e-5
    assert Hh.rel_err(Wk.grad, Wko.grad) < 5e-5
    for x, y in zip(Wax, Waxo):
        assert x.grad.shape == (1, Hh.H, Hh.DH, A16)
        assert Hh.rel_err(x.grad, y.grad) < 5e-5


@pytest.mark.parametrize("cos_abs", [0, 1])
def test_sixteen_angle_bins_match_the_port_of_the_kernel_text(cos_abs):
    """The float32 scalar port of the reference kernels with ANGLE_ENC_DIM 16, ANGLE_RANGE 9: the branch that sums
    all bins."""
    import crystalframer_amd as cf
    P = Hh.make_problem(num_crystals=8, atoms_hi=5, seed=9)
    W16 = _weights16(P, seed=6)
    fr = [g(f) for f in P.frames]
    z, psi = cf.RealEncodingWithFramedProjFuncCUDA.apply(
        g(P.a), g(P.rpos), None, g(P.tvecs), P.batch.to(dev()), P.edges.to(dev()), 64, Hh.DIST_MAX, 1.0, g(P.W_k),
        g(W16[0]), g(W16[1]), g(W16[2]), fr[0], fr[1], fr[2], A16, 1.0, cos_abs, 1.5, 6.0, g(P.rvlen), CUT)
    p = CO.make_params(A=A16, angle_wscale=1.0, cos_abs=cos_abs, dist_coef=1.5, angle_coef=6.0, cutoff_radius=CUT)
    assert p.angle_range == 9
    zc, psic, _ = CO.pe_forward(p, P.a, P.rpos, P.tvecs, P.rvlen, P.batch, P.edges, P.W_k[0], W16, P.frames, "f32")
    assert Hh.rel_err(z, zc) < 2e-5
    assert Hh.rel_err(psi, psic) < 5e-5


@pytest.mark.parametrize("cos_abs", [0, 1])
@pytest.mark.parametrize("wscale,sizes", [(1.0, (1, 6)), (2.0, (1, 6)), (1.0, (20, 40))])
def test_sixteen_angle_bins_fused_core(cos_abs, wscale, sizes):
    """The fused attention core with the 16-bin basis (every image adds all 16 basis values per axis into the
    item's histogram of 64 + 3 x 16 words) against the composition of the float64 oracles, whole angle basis and
    the core's default +-5 sigma distance window; rows of up to 40 pairs (several groups: the running softmax
    rescales the histogram) and one-atom crystals."""
    from crystalframer_amd import cuda_funcs as F
    P = Hh.make_problem(num_crystals=10 if sizes[1] < 10 else 4, atoms_lo=sizes[0], atoms_hi=sizes[1],
                        len_lo=3.0 if sizes[1] < 10 else 2.5, len_hi=8.0, seed=150 + cos_abs)
    if sizes[1] >= 10:
        P.q = P.q * 4.0
    W16 = _weights16(P, seed=7)
    cd, ca = 1.5, 6.0
    names = ("q", "k", "v", "a", "Wk", "W1", "W2", "W3")
    src = dict(q=P.q, k=P.k, v=P.v, a=P.a, Wk=P.W_k, W1=W16[0], W2=W16[1], W3=W16[2])
    lv = {n: g(src[n]).requires_grad_(True) for n in names}
    out, fr = F.PeriodicAttentionCoreHIP.apply(
        lv["q"], lv["k"], lv["v"], lv["a"], g(P.rpos), g(P.tvecs), P.batch.to(dev()), P.edges.to(dev()), 64, Hh.DIST_MAX,
        1.0, lv["Wk"], lv["W1"], lv["W2"], lv["W3"], A16, wscale, cos_abs, cd, ca, g(P.rvlen), CUT,
        torch.stack([g(f) for f in P.frames], 0))
    lo = {n: src[n].clone().requires_grad_(True) for n in names}
    zo, psio = TO.framed_pe(lo["a"], P.rpos, P.tvecs, P.batch, P.edges, lo["Wk"], [lo["W1"], lo["W2"], lo["W3"]], P.frames,
                            K=64, A=A16, angle_wscale=wscale, cos_abs=cos_abs, c_dist=cd, c_angle=ca, rvlen=P.rvlen,
                            cutoff_radius=CUT, windows=(11, None))
    oo, _ = TO.softmax_attention(lo["q"], lo["k"], lo["v"], zo, psio, P.batch, P.edges)
    assert torch.isfinite(out).all()
    assert Hh.rel_err(out, oo) < 2e-5 and Hh.elem_err(out, oo, rtol=1e-4, atol_frac=1e-5) <= 1.0
    gout = torch.randn(P.N, Hh.H, Hh.DH, generator=torch.Generator().manual_seed(3), dtype=torch.float64)
    (out * g(gout)).sum().backward()
    (oo * gout).sum().backward()
    for n in names:
        assert lv[n].grad.shape == lo[n].grad.shape, n
        assert Hh.rel_err(lv[n].grad, lo[n].grad) < 1e-4, n


def test_lightweight_model_forward_backward_matches_cpu_model(core_mode):
    """Two layers with the lightweight setting against the float64 CPU model, output and every parameter gradient,
    through the fused core (whole bases) and through the two-step operators (the reference's windows)."""
    import crystalframer_amd as cf
    from crystalframer_amd import latticeformer, params, synthetic
    mp = params.ModelParams(num_layers=2, value_pe_angle_real=A16, value_pe_angle_wscale=1.0, value_pe_dist_coef=1.5,
                            value_pe_angle_coef=6.0, symm_break_noise=0.0)
    cb = synthetic.make_batch(8, atoms="uniform", atoms_lo=1, atoms_hi=6, len_lo=3.0, len_hi=9.0, ang_lo=65.0,
                              ang_hi=115.0, seed=12)
    torch.manual_seed(0)
    model = latticeformer.Latticeformer(mp).to(dev())
    for layer in model.encoder.layers:
        layer.self_attn.frame_sink = []
    target = torch.linspace(-1, 1, cb.num_crystals, device=dev())[:, None]
    out = model(cb.to(dev()))
    torch.nn.functional.mse_loss(out, target).backward()
    torch.cuda.synchronize()
    sd = {k: v.detach().cpu().double() for k, v in model.state_dict().items()}
    leaves = {k: v.clone().requires_grad_("scale" not in k) for k, v in sd.items()}
    assert leaves["encoder.layers.0.self_attn.proj_angle1"].shape[-1] == A16
    frames = [[f.detach().cpu().double() for f in layer.self_attn.frame_sink[0]] for layer in model.encoder.layers]
    ref = cpu_model.model_forward(leaves, cb, mp, dtype=torch.float64, frames_per_layer=frames, windows=core_mode)
    torch.nn.functional.mse_loss(ref, target.cpu().double()).backward()
    assert Hh.rel_err(out, ref) < 1e-4
    checked = 0
    for name, p in model.named_parameters():
        if p.grad is None:
            continue
        assert Hh.rel_err(p.grad, leaves[name].grad) < 1e-4, name
        checked += 1
    assert checked >= 20
