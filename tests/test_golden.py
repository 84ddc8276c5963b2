"""The committed golden vectors (tests/golden/framed_pe_small.npz, written by
tests/golden/make_golden.py from the float64 tensor oracle): the scalar C oracle must reproduce them
on the CPU, the HIP kernels on the GPU."""
import os

import numpy as np
import pytest
import torch

import helpers as Hh
from oracle import c_oracle as CO
from oracle import torch_oracle as TO

GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "framed_pe_small.npz")
CUT = -3.5


def load():
    d = np.load(GOLD, allow_pickle=False)
    return {k: torch.from_numpy(d[k]) for k in d.files}


def test_c_oracle_reproduces_golden_vectors():
    G = load()
    p = CO.make_params(cutoff_radius=CUT)
    W_ax = [G["W_ax"][i] for i in range(3)]
    frames = [G["frames"][i] for i in range(3)]
    z, psi, _ = CO.pe_forward(p, G["a"], G["rpos"], G["tvecs"], G["rvlen"], G["batch"], G["edges"], G["W_k"][0], W_ax,
                              frames, "f64")
    assert Hh.rel_err(z, G["z"]) < 1e-12
    assert Hh.rel_err(psi, G["psi"]) < 1e-12
    ga, gWd, gWa = CO.pe_backward(p, G["a"], G["rpos"], G["tvecs"], G["rvlen"], G["batch"], G["edges"], G["W_k"][0],
                                  W_ax, frames, z, G["gz"], G["gpsi"], "f64")
    assert Hh.rel_err(ga, G["ga"]) < 1e-10
    assert Hh.rel_err(gWd, G["gW_k"][0]) < 1e-10
    for ax in range(3):
        assert Hh.rel_err(gWa[ax], G["gW_ax"][ax][0]) < 1e-10
    f1, f2 = CO.frame_axes(p, G["q"], G["k"], G["a"], G["rpos"], G["tvecs"], G["rvlen"], G["batch"], G["edges"], "f64")
    clear = (G["gap1"] > 1e-9) & (G["gap2"] > 1e-9)
    assert clear.double().mean() > 0.9
    assert (f1 - G["frame1"])[G["gap1"] > 1e-9].abs().max() < 1e-12
    assert (f2 - G["frame2max"])[clear].abs().max() < 1e-12
    out, prob = CO.dpa_forward(G["q"], G["k"], G["v"], G["z"], G["psi"], G["edges"], "f64")
    assert Hh.rel_err(out, G["attn_out"]) < 1e-12
    assert Hh.rel_err(prob, G["attn_prob"]) < 1e-12
    # and the tensor oracle still gives what it gave when the vectors were written
    z2, psi2 = TO.framed_pe(G["a"], G["rpos"], G["tvecs"], G["batch"], G["edges"], G["W_k"], W_ax, frames, K=64, A=64,
                            cos_abs=0, c_dist=1.0, c_angle=1.0, rvlen=G["rvlen"], cutoff_radius=CUT,
                            windows="reference")
    assert Hh.rel_err(z2, G["z"]) < 1e-13 and Hh.rel_err(psi2, G["psi"]) < 1e-13


@pytest.mark.gpu
def test_hip_kernels_reproduce_golden_vectors():
    import crystalframer_amd as cf
    KM = cf.KernelManager
    saved = (KM.SYMM_BREAK_NOISE, KM.PRUNE_LOG2, KM.WINDOW_MODE)
    KM.SYMM_BREAK_NOISE, KM.PRUNE_LOG2, KM.WINDOW_MODE = 0.0, 24.0, 0
    try:
        G = load()
        dev = torch.device("cuda:0")
        f = lambda t: t.to(dtype=torch.float32, device=dev)
        a = f(G["a"]).requires_grad_(True)
        Wk = f(G["W_k"]).requires_grad_(True)
        Wax = [f(G["W_ax"][i]).requires_grad_(True) for i in range(3)]
        fr = [f(G["frames"][i]) for i in range(3)]
        batch, edges = G["batch"].to(dev), G["edges"].to(dev)
        z, psi = cf.RealEncodingWithFramedProjFuncCUDA.apply(
            a, f(G["rpos"]), None, f(G["tvecs"]), batch, edges, 64, Hh.DIST_MAX, 1.0, Wk, Wax[0], Wax[1], Wax[2],
            fr[0], fr[1], fr[2], 64, 4.0, 0, 1.0, 1.0, f(G["rvlen"]), CUT)
        assert Hh.rel_err(z, G["z"]) < 2e-5
        assert Hh.rel_err(psi, G["psi"]) < 2e-5
        ((z * f(G["gz"])).sum() + (psi * f(G["gpsi"])).sum()).backward()
        assert Hh.rel_err(a.grad, G["ga"]) < 5e-5
        assert Hh.rel_err(Wk.grad, G["gW_k"]) < 5e-5
        for ax in range(3):
            assert Hh.rel_err(Wax[ax].grad, G["gW_ax"][ax]) < 5e-5
        args = (f(G["q"]), f(G["k"]), None, f(G["a"]), f(G["rpos"]), None, f(G["tvecs"]), batch, edges, 64,
                Hh.DIST_MAX, 1.0, f(G["rvlen"]), CUT)
        f1 = cf.ComputeFrame1MaximumMethodCUDA.apply(*args[:12], *args[12:])
        f2 = cf.ComputeFrame2MaximumMethodCUDA.apply(*args[:12], f1, *args[12:])
        clear1 = G["gap1"] > 1e-4
        clear2 = clear1 & (G["gap2"] > 1e-4)
        assert (f1.cpu().double() - G["frame1"])[clear1].abs().max() < 1e-5
        assert (f2.cpu().double() - G["frame2max"])[clear2].abs().max() < 1e-5
        out = cf.FusedDotProductAttentionCUDA.apply(f(G["q"]), f(G["k"]), f(G["v"]), f(G["z"]), f(G["psi"]), batch, edges)
        assert Hh.rel_err(out, G["attn_out"]) < 2e-5
    finally:
        KM.SYMM_BREAK_NOISE, KM.PRUNE_LOG2, KM.WINDOW_MODE = saved
