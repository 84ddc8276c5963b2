"""Distance bases of another width than the default: value_pe_dist_wscale != 1.  The reference derives the window of
its kernels from the scale, LENGTH_RANGE = ceil(8 wscale + 1) bins starting at int((d - 4 sigma) / interval - 1), and
evaluates the whole basis when that leaves at most 8 of the 64 bins out (models/cuda_funcs/kernel_manager.py:146,
models/kernels/real_enc_frame_proj_fwd_length.cu:139-160).  The kernels here are compiled for the widths of scale 1
and once more for a width known at run time; scales that give an even width (0.6: 6 bins), an odd one (1.7: 15) and
the whole basis (8.0) go through that instantiation.

Tolerances as for the default scale: operators 2e-5 forward, 5e-5 gradients against the float64 oracle with the same
window; the fused core 2e-5 / 1e-4, and 1e-4 against the untruncated bases in its default mode."""
import math

import pytest
import torch

import helpers as Hh
from oracle import cpu_model
from oracle import torch_oracle as TO

pytestmark = pytest.mark.gpu
CUT = -3.5
SCALES = [0.6, 1.7, 8.0]


@pytest.fixture(autouse=True)
def _defaults():
    import crystalframer_amd as cf
    KM = cf.KernelManager
    names = ("SYMM_BREAK_NOISE", "PRUNE_LOG2", "WINDOW_MODE", "CORE_WINDOW_MODE", "GRAD_COEF_QUIRK", "LATTICE_RANGE",
             "MINIMUM_RANGE", "SAVE_HISTOGRAMS", "SECOND_STREAM")
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


@pytest.mark.parametrize("wscale", SCALES)
@pytest.mark.parametrize("save_histograms", [True, False])
def test_operators_with_another_distance_scale(wscale, save_histograms):
    import crystalframer_amd as cf
    cf.KernelManager.SAVE_HISTOGRAMS = save_histograms
    P = Hh.make_problem(num_crystals=10, atoms_hi=6, seed=160)
    cd, ca = 0.8, 1.2
    a = g(P.a).requires_grad_(True)
    Wk = g(P.W_k).requires_grad_(True)
    Wax = [g(w).requires_grad_(True) for w in P.W_ax]
    fr = [g(f) for f in P.frames]
    z, psi = cf.RealEncodingWithFramedProjFuncCUDA.apply(
        a, g(P.rpos), None, g(P.tvecs), P.batch.to(dev()), P.edges.to(dev()), 64, Hh.DIST_MAX, wscale, Wk, Wax[0],
        Wax[1], Wax[2], fr[0], fr[1], fr[2], 64, 4.0, 0, cd, ca, g(P.rvlen), CUT)
    ao = P.a.clone().requires_grad_(True)
    Wko = P.W_k.clone().requires_grad_(True)
    Waxo = [w.clone().requires_grad_(True) for w in P.W_ax]
    zo, psio = TO.framed_pe(ao, P.rpos, P.tvecs, P.batch, P.edges, Wko, Waxo, P.frames, wscale=wscale, c_dist=cd,
                            c_angle=ca, rvlen=P.rvlen, cutoff_radius=CUT, windows="reference")
    assert Hh.rel_err(z, zo) < 2e-5
    assert Hh.rel_err(psi, psio) < 2e-5 and Hh.elem_err(psi, psio, atol_frac=1e-5) <= 1.0
    ((z * g(P.gz)).sum() + (psi * g(P.gpsi)).sum()).backward()
    ((zo * P.gz).sum() + (psio * P.gpsi).sum()).backward()
    assert Hh.rel_err(a.grad, ao.grad) < 5e-5
    assert Hh.rel_err(Wk.grad, Wko.grad) < 5e-5
    for x, y in zip(Wax, Waxo):
        assert Hh.rel_err(x.grad, y.grad) < 5e-5


def _core(P, wscale, A=64):
    from crystalframer_amd import cuda_funcs as F
    names = ("q", "k", "v", "a", "Wk", "W1", "W2", "W3")
    src = dict(q=P.q, k=P.k, v=P.v, a=P.a, Wk=P.W_k, W1=P.W_ax[0], W2=P.W_ax[1], W3=P.W_ax[2])
    lv = {n: g(src[n]).requires_grad_(True) for n in names}
    out, _ = F.PeriodicAttentionCoreHIP.apply(
        lv["q"], lv["k"], lv["v"], lv["a"], g(P.rpos), g(P.tvecs), P.batch.to(dev()), P.edges.to(dev()), 64, Hh.DIST_MAX,
        wscale, lv["Wk"], lv["W1"], lv["W2"], lv["W3"], A, 4.0, 0, 0.8, 1.2, g(P.rvlen), CUT,
        torch.stack([g(f) for f in P.frames], 0))
    return out, lv, src, names


def _oracle(P, src, names, wscale, windows):
    lo = {n: src[n].clone().requires_grad_(True) for n in names}
    zo, psio = TO.framed_pe(lo["a"], P.rpos, P.tvecs, P.batch, P.edges, lo["Wk"], [lo["W1"], lo["W2"], lo["W3"]], P.frames,
                            wscale=wscale, c_dist=0.8, c_angle=1.2, rvlen=P.rvlen, cutoff_radius=CUT, windows=windows)
    oo, _ = TO.softmax_attention(lo["q"], lo["k"], lo["v"], zo, psio, P.batch, P.edges)
    return oo, lo


@pytest.mark.parametrize("wscale", SCALES)
def test_fused_core_with_another_distance_scale(wscale):
    """The 4-sigma window of the scale (the reference's rule) against the oracle with the same window, angle basis
    untruncated; then the core's default 5-sigma window against the untruncated bases."""
    import crystalframer_amd as cf
    KM = cf.KernelManager
    P = Hh.make_problem(num_crystals=10, atoms_hi=6, seed=161)
    gout = torch.randn(P.N, Hh.H, Hh.DH, generator=torch.Generator().manual_seed(4), dtype=torch.float64)
    KM.CORE_WINDOW_MODE = 0
    out, lv, src, names = _core(P, wscale)
    oo, lo = _oracle(P, src, names, wscale, (math.ceil(8 * wscale + 1), None))
    assert Hh.rel_err(out, oo) < 2e-5
    (out * g(gout)).sum().backward()
    (oo * gout).sum().backward()
    for n in names:
        assert Hh.rel_err(lv[n].grad, lo[n].grad) < 1e-4, n
    KM.CORE_WINDOW_MODE = 1
    out, lv, src, names = _core(P, wscale)
    oo, lo = _oracle(P, src, names, wscale, "full")
    assert Hh.rel_err(out, oo) < 1e-4
    (out * g(gout)).sum().backward()
    (oo * gout).sum().backward()
    for n in names:
        assert Hh.rel_err(lv[n].grad, lo[n].grad) < 1e-4, n


def test_model_with_another_distance_scale(core_mode):
    from crystalframer_amd import latticeformer, params, synthetic
    mp = params.ModelParams(num_layers=2, value_pe_dist_wscale=1.5, symm_break_noise=0.0)
    cb = synthetic.make_batch(8, atoms="uniform", atoms_lo=1, atoms_hi=6, len_lo=3.0, len_hi=9.0, ang_lo=65.0,
                              ang_hi=115.0, seed=14)
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
