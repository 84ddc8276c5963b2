"""End-to-end parity of the model (attention layer, encoder, pooling, head) on the GPU against the
float64 CPU restatement, forward and parameter gradients."""
import pytest
import torch

import helpers as Hh
from oracle import cpu_model

pytestmark = pytest.mark.gpu


def _run(mp, cb, seed=0, passes=1, windows="reference"):
    import crystalframer_amd as cf
    from crystalframer_amd import latticeformer
    KM = cf.KernelManager
    KM.SYMM_BREAK_NOISE = 0.0
    dev = torch.device("cuda:0")
    torch.manual_seed(seed)
    model = latticeformer.Latticeformer(mp).to(dev)
    for layer in model.encoder.layers:
        layer.self_attn.frame_sink = []
        layer.self_attn.grad_sink = {}
    target = torch.linspace(-1, 1, cb.num_crystals, device=dev)[:, None]
    for _ in range(passes):
        # the first training-mode pass measures and stores the normalisation of alpha with framework
        # ops; later passes take the fused split / scaling / Gaussian-coefficient launch
        model.zero_grad(set_to_none=True)
        for layer in model.encoder.layers:
            layer.self_attn.frame_sink.clear()
        out = model(cb.to(dev))
        loss = torch.nn.functional.mse_loss(out, target)
        loss.backward()
    torch.cuda.synchronize()
    sd = {k: v.detach().cpu().double() for k, v in model.state_dict().items()}
    leaves = {k: v.clone().requires_grad_("scale" not in k) for k, v in sd.items()}
    frames = None
    if mp.value_pe_angle_real > 0:
        frames = [[f.detach().cpu().double() for f in layer.self_attn.frame_sink[0]] for layer in model.encoder.layers]
    ref, auxes = cpu_model.model_forward(leaves, cb, mp, dtype=torch.float64, frames_per_layer=frames, windows=windows,
                                         return_aux=True)
    for aux in auxes:
        for n in ("qs", "k", "v", "a"):
            aux[n].retain_grad()
    ref_loss = torch.nn.functional.mse_loss(ref, target.cpu().double())
    ref_loss.backward()
    model.oracle_auxes = auxes
    return model, out, ref, leaves


@pytest.mark.parametrize("angle_bins,passes", [(64, 1), (0, 1), (64, 2)])
def test_model_forward_backward_matches_cpu_oracle(angle_bins, passes, core_mode):
    from crystalframer_amd import params, synthetic
    mp = params.ModelParams(num_layers=2, value_pe_angle_real=angle_bins, symm_break_noise=0.0)
    cb = synthetic.make_batch(8, atoms="uniform", atoms_lo=1, atoms_hi=6, len_lo=3.0, len_hi=9.0,
                              ang_lo=65.0, ang_hi=115.0, seed=11)
    model, out, ref, leaves = _run(mp, cb, passes=passes, windows=core_mode)
    assert Hh.rel_err(out, ref) < 1e-4
    Hh.check_model_gradients(model, leaves, model.oracle_auxes, tol=1e-4, min_checked=20)
    # the first training-mode forward stored the normalisation of alpha
    for layer in model.encoder.layers:
        assert float(layer.self_attn.gauss_scale[0]) > 0


def test_model_frames_agree_with_oracle_frames(core_mode):
    """The frames the model used are the oracle's wherever the winner is clear."""
    from crystalframer_amd import params, synthetic
    from oracle import torch_oracle as TO
    import math
    mp = params.ModelParams(num_layers=1, symm_break_noise=0.0)
    cb = synthetic.make_batch(8, atoms="uniform", atoms_lo=2, atoms_hi=6, len_lo=3.0, len_hi=9.0,
                              ang_lo=65.0, ang_hi=115.0, seed=13)
    model, out, ref, leaves = _run(mp, cb, windows=core_mode)
    sd = {k: v.detach() for k, v in leaves.items()}
    lat = params.LatticeformerParams().parseFromArgs(mp).getLayerParameters(0)
    pos, tv = cb.pos.double(), cb.trans_vec.double()
    edges, rpos, recip, _ = TO.geometry(pos, tv, cb.sizes.tolist())
    geo = dict(edges=edges, rpos=rpos, tvecs=tv, rvlen=recip.norm(dim=-1), batch=cb.batch)
    x = torch.nn.functional.linear(cb.x.double(), sd["input_embeddings.weight"])
    _, aux = cpu_model.attention_layer(x, sd, "encoder.layers.0.self_attn.", geo, lat, return_aux=True)
    q = aux["q"] / math.sqrt(16)
    f1, f2, gap1, gap2 = TO.frame_axes_max(q, aux["k"], aux["a"], rpos, tv, cb.batch, edges, rvlen=geo["rvlen"],
                                           cutoff_radius=-3.5, return_gaps=True)
    used = model.encoder.layers[0].self_attn.frame_sink[0]
    clear = (gap1 > 1e-4) & (gap2 > 1e-4)
    assert clear.double().mean() > 0.9
    assert (used[0].cpu().double() - f1)[clear].abs().max() < 1e-4


@pytest.mark.parametrize("fixed_order", [True, False])
def test_training_step_as_hip_graph_matches_eager_on_every_replay(fixed_order):
    """The whole training step (geometry, forward, loss, backward, AdamW) captured as one HIP graph:
    every replay is compared with an eager twin of the same model, with eager work and
    synchronisations between the replays.  With the weight gradients of the linear layers summed in a fixed order
    (KernelManager.DETERMINISTIC_WEIGHT_GRADIENTS, the default) every kernel of the step adds in a fixed order and
    the twins stay bit-equal; with float atomics they drift apart as bounded below."""
    import crystalframer_amd as cf
    from crystalframer_amd import latticeformer, params, synthetic
    KM = cf.KernelManager
    dev = torch.device("cuda:0")
    saved = (KM.SYMM_BREAK_NOISE, KM.NOISE_SEED, KM.NOISE_SEED_DEVICE)
    saved_order = KM.DETERMINISTIC_WEIGHT_GRADIENTS
    KM.DETERMINISTIC_WEIGHT_GRADIENTS = fixed_order
    mp = params.ModelParams(num_layers=2)
    cb = synthetic.make_batch(24, atoms="uniform", atoms_lo=1, atoms_hi=9, len_lo=3.0, len_hi=9.0,
                              ang_lo=65.0, ang_hi=115.0, seed=21).to(dev)
    assert cb.num_pairs > 0          # host-known pair count: the geometry needs no device read
    target = torch.linspace(-1, 1, cb.num_crystals, device=dev)[:, None]

    def twin():
        torch.manual_seed(5)
        model = latticeformer.Latticeformer(mp).to(dev)
        model.train()
        opt = torch.optim.AdamW(model.parameters(), lr=1e-3, capturable=True)
        seed_word = torch.zeros(1, dtype=torch.int64, device=dev)
        loss_out = torch.zeros((), device=dev)

        def step():
            KM.NOISE_SEED_DEVICE = seed_word
            opt.zero_grad(set_to_none=True)
            loss = torch.nn.functional.mse_loss(model(cb), target)
            loss.backward()
            opt.step()
            loss_out.copy_(loss.detach())
        return model, step, loss_out

    try:
        KM.SYMM_BREAK_NOISE, KM.NOISE_SEED = 1e-5, 99
        model_e, step_e, loss_e = twin()
        model_g, step_g, loss_g = twin()
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            for _ in range(3):
                step_g()
        torch.cuda.current_stream().wait_stream(side)
        for _ in range(3):
            step_e()
        torch.cuda.synchronize()
        assert abs(float(loss_e) - float(loss_g)) < 1e-4 * abs(float(loss_e))
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            step_g()
        junk = torch.randn(512, 512, device=dev)
        for replay in range(5):
            step_e()
            graph.replay()
            torch.cuda.synchronize()
            le, lg = float(loss_e), float(loss_g)
            assert abs(le - lg) < 2e-4 * abs(le), (replay, le, lg)
            assert le == lg or not fixed_order, (replay, le, lg)
            junk = torch.tanh(junk @ junk / 512.0)          # eager work between the replays
            assert torch.isfinite(junk).all()
        # With float atomics the twins are not bit-equal, and AdamW's first steps move every element by about lr
        # whatever the size of its gradient, so an element whose tiny gradient differs in the last bits (or in sign)
        # drifts by up to 2 lr per step.  Bound: two such steps for any element, a hundredth of a step on average.
        lr = 1e-3
        for (n, pe), (_, pg) in zip(model_e.named_parameters(), model_g.named_parameters()):
            diff = (pg.detach() - pe.detach()).abs()
            if fixed_order:
                assert float(diff.max()) == 0.0, n
            assert float(diff.max()) <= 4 * lr, n
            assert float(diff.mean()) <= 0.02 * lr, n
    finally:
        KM.SYMM_BREAK_NOISE, KM.NOISE_SEED, KM.NOISE_SEED_DEVICE = saved
        KM.DETERMINISTIC_WEIGHT_GRADIENTS = saved_order


def test_bridged_encoder_equals_the_modules_own_forward():
    """The encoder as attention cores joined by the layer bridge against the same model run module by
    module (out_proj, residual, feed-forward block, next input projection as separate calls): outputs and
    gradients agree to float32 rounding, in training mode and under no_grad in eval mode."""
    import crystalframer_amd as cf
    from crystalframer_amd import encoder, latticeformer, params, synthetic
    cf.KernelManager.SYMM_BREAK_NOISE = 0.0
    dev = torch.device("cuda:0")
    mp = params.ModelParams(num_layers=3, symm_break_noise=0.0)
    cb = synthetic.make_batch(9, atoms="uniform", atoms_lo=1, atoms_hi=7, len_lo=3.0, len_hi=9.0,
                              ang_lo=65.0, ang_hi=115.0, seed=17).to(dev)
    torch.manual_seed(3)
    model = latticeformer.Latticeformer(mp).to(dev)
    model.train()
    model(cb).sum().backward()          # first pass: stores the normalisation of alpha (module path)
    assert model.encoder._bridge_ready(torch.zeros(1, mp.model_dim, device=dev))
    results = []
    for bridged in (True, False):
        encoder.FUSED_LAYER_BRIDGE = bridged
        try:
            model.zero_grad(set_to_none=True)
            out = model(cb)
            (out.square().sum()).backward()
            grads = {n: p.grad.clone() for n, p in model.named_parameters() if p.grad is not None}
            model.eval()
            with torch.no_grad():
                out_eval = model(cb)
            model.train()
        finally:
            encoder.FUSED_LAYER_BRIDGE = True
        results.append((out.detach(), out_eval, grads))
    (o1, e1, g1), (o2, e2, g2) = results
    assert Hh.rel_err(o1, o2.double()) < 1e-5 and Hh.rel_err(e1, e2.double()) < 1e-5
    assert Hh.rel_err(e1, o1.double()) < 1e-5          # no dropout: eval equals training output
    assert g1.keys() == g2.keys() and len(g1) >= 30
    for n in g1:
        assert Hh.rel_err(g1[n], g2[n].double()) < 1e-4, n


def test_gradients_accumulate_over_two_passes_and_match_the_single_stream_path():
    """Weight gradients that leave for the second stream in the middle of the backward pass (those of the
    layers behind a lattice backward) must end up where autograd accumulates: a second pass without
    zero_grad doubles every gradient, and the pass with everything on one stream gives the same values."""
    import crystalframer_amd as cf
    from crystalframer_amd import latticeformer, params, synthetic
    KM = cf.KernelManager
    saved = (KM.SYMM_BREAK_NOISE, KM.SECOND_STREAM)
    KM.SYMM_BREAK_NOISE = 0.0
    dev = torch.device("cuda:0")
    mp = params.ModelParams(num_layers=3, symm_break_noise=0.0)
    cb = synthetic.make_batch(12, atoms="uniform", atoms_lo=1, atoms_hi=8, len_lo=3.0, len_hi=9.0,
                              ang_lo=65.0, ang_hi=115.0, seed=23).to(dev)
    torch.manual_seed(5)
    model = latticeformer.Latticeformer(mp).to(dev)
    model.train()
    model(cb).sum().backward()          # stores the normalisation of alpha
    try:
        grads = {}
        for second in (True, False):
            KM.SECOND_STREAM = second
            model.zero_grad(set_to_none=True)
            model(cb).square().sum().backward()
            once = {n: p.grad.clone() for n, p in model.named_parameters() if p.grad is not None}
            model(cb).square().sum().backward()          # accumulates into the existing .grad
            twice = {n: p.grad.clone() for n, p in model.named_parameters() if p.grad is not None}
            assert once.keys() == twice.keys() and len(once) >= 30
            for n in once:
                assert Hh.rel_err(twice[n], 2.0 * once[n].double()) < 2e-5, (second, n)
            grads[second] = once
        for n in grads[True]:
            assert Hh.rel_err(grads[True][n], grads[False][n].double()) < 2e-5, n
    finally:
        KM.SYMM_BREAK_NOISE, KM.SECOND_STREAM = saved


_CAPTURE_FIRST = r'''
import sys, torch
sys.path.insert(0, "tests"); sys.path.insert(0, ".")
import helpers as Hh
import crystalframer_amd as cf
from crystalframer_amd import cuda_funcs
cf.KernelManager.SYMM_BREAK_NOISE = 0.0
dev = torch.device("cuda:0")
P = Hh.make_problem(num_crystals=6, atoms_hi=5, seed=3)
g = lambda t: t.to(dtype=torch.float32, device=dev)
a = g(P.a).requires_grad_(True)
Wk = g(P.W_k).requires_grad_(True)
Wax = [g(w).requires_grad_(True) for w in P.W_ax]
fr = [g(f) for f in P.frames]
rpos, tv, rv, batch, edges = g(P.rpos), g(P.tvecs), g(P.rvlen), P.batch.to(dev), P.edges.to(dev)
gz, gpsi = g(P.gz), g(P.gpsi)
cuda_funcs.edge_schedule(edges, P.N)          # framework arithmetic only: no library call so far
torch.cuda.synchronize()

def run():
    z, psi = cf.RealEncodingWithFramedProjFuncCUDA.apply(
        a, rpos, None, tv, batch, edges, 64, 14.0, 1.0, Wk, Wax[0], Wax[1], Wax[2], fr[0], fr[1], fr[2],
        64, 4.0, 0, 1.0, 1.0, rv, -3.5)
    return torch.autograd.grad([z, psi], [a, Wk] + Wax, [gz, gpsi])

side = torch.cuda.Stream()
graph = torch.cuda.CUDAGraph()
with torch.cuda.stream(side):
    with torch.cuda.graph(graph, stream=side):      # the library's first calls of this process are captured
        out = run()
for _ in range(2):
    graph.replay()
torch.cuda.synchronize()
captured = [o.clone() for o in out]
eager = run()
torch.cuda.synchronize()
for c, e in zip(captured, eager):
    assert torch.isfinite(c).all()
    err = float((c - e).abs().max() / e.abs().max().clamp_min(1e-30))
    assert err < 1e-5, err
print("CAPTURE-FIRST-OK")
'''


def test_the_first_backward_of_a_process_can_be_captured():
    """The library creates its second stream on first use; that first use may be under graph capture."""
    import os
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    res = subprocess.run([sys.executable, "-c", _CAPTURE_FIRST], cwd=root, capture_output=True, text=True, timeout=110)
    assert res.returncode == 0 and "CAPTURE-FIRST-OK" in res.stdout, res.stdout[-2000:] + res.stderr[-4000:]


def test_crystal_indices_with_an_offset_give_the_same_output():
    """The reference subtracts batch[0] (a chunk of a split batch does not start at 0); a batch that is known
    to start at 0 skips that subtraction."""
    from crystalframer_amd import latticeformer, params, synthetic
    dev = torch.device("cuda:0")
    mp = params.ModelParams(num_layers=2, symm_break_noise=0.0)
    cb = synthetic.make_batch(7, atoms="uniform", atoms_lo=1, atoms_hi=6, len_lo=3.0, len_hi=9.0,
                              ang_lo=65.0, ang_hi=115.0, seed=31)
    assert cb.zero_based
    torch.manual_seed(1)
    model = latticeformer.Latticeformer(mp).to(dev)
    model.train()
    model(cb.to(dev))
    model.eval()
    with torch.no_grad():
        ref = model(cb.to(dev))
        shifted = synthetic.CrystalBatch(cb.x, cb.pos, cb.batch + 5, cb.trans_vec, cb.sizes).to(dev)
        assert not shifted.zero_based
        out = model(shifted)
    assert torch.equal(out, ref)


def test_a_bare_batch_object_with_the_reference_fields_only():
    """What the reference's data loader hands the model (dataloaders/dataset_latticeformer.py:32-37): an object with
    x, pos, batch, trans_vec and sizes and nothing else (no host-known pair count, no zero-based flag).  Same output
    and gradients as the CrystalBatch that carries the extras."""
    import types
    from crystalframer_amd import latticeformer, params, synthetic
    dev = torch.device("cuda:0")
    mp = params.ModelParams(num_layers=2, symm_break_noise=0.0)
    cb = synthetic.make_batch(7, atoms="uniform", atoms_lo=1, atoms_hi=6, len_lo=3.0, len_hi=9.0,
                              ang_lo=65.0, ang_hi=115.0, seed=33).to(dev)
    bare = types.SimpleNamespace(x=cb.x, pos=cb.pos, batch=cb.batch, trans_vec=cb.trans_vec, sizes=cb.sizes)
    torch.manual_seed(2)
    model = latticeformer.Latticeformer(mp).to(dev)
    model.train()
    model(cb)                      # stores the normalisation of alpha
    results = []
    for data in (cb, bare):
        model.zero_grad(set_to_none=True)
        out = model(data)
        out.square().sum().backward()
        results.append((out.detach().clone(), {n: p.grad.clone() for n, p in model.named_parameters() if p.grad is not None}))
    assert torch.equal(results[0][0], results[1][0])
    for n, gr in results[0][1].items():
        assert Hh.rel_err(results[1][1][n], gr) < 1e-6, n


def test_hooked_parameter_and_reused_weight_get_complete_gradients():
    """Deferred weight gradients must not be visible as zeros: a parameter with a tensor hook or a
    post-accumulate hook is not deferred (its hook sees the finished gradient), and a weight used by two
    projections of one pass receives the sum of both products."""
    import crystalframer_amd as cf
    dev = torch.device("cuda:0")
    gen = torch.Generator().manual_seed(3)
    x1 = torch.randn(300, 128, generator=gen).to(dev)
    x2 = torch.randn(300, 128, generator=gen).to(dev)
    W0 = torch.randn(64, 128, generator=gen)
    b0 = torch.randn(64, generator=gen)
    gy = torch.randn(300, 64, generator=gen).to(dev)

    def reference():
        W = W0.double().requires_grad_(True)
        b = b0.double().requires_grad_(True)
        y = torch.nn.functional.linear(x1.cpu().double(), W, b) + 2.0 * torch.nn.functional.linear(x2.cpu().double(), W, b)
        (y * gy.cpu().double()).sum().backward()
        return W.grad, b.grad

    gW_ref, gb_ref = reference()
    for kind in ("plain", "tensor_hook", "post_accumulate_hook"):
        W = W0.to(dev).requires_grad_(True)
        b = b0.to(dev).requires_grad_(True)
        seen = {}
        if kind == "tensor_hook":
            W.register_hook(lambda g: seen.setdefault("calls", []).append(g.detach().clone()))
        elif kind == "post_accumulate_hook":
            W.register_post_accumulate_grad_hook(lambda p: seen.setdefault("calls", []).append(p.grad.detach().clone()))
        y = cf.cuda_funcs.linear(x1, W, b) + 2.0 * cf.cuda_funcs.linear(x2, W, b)
        (y * gy).sum().backward()
        torch.cuda.synchronize()
        assert Hh.rel_err(W.grad, gW_ref) < 1e-5, kind
        assert Hh.rel_err(b.grad, gb_ref) < 1e-5, kind
        if kind == "tensor_hook":
            # the engine sums the two uses before it calls the hook: what the hook sees is the gradient
            assert len(seen["calls"]) == 1
            assert Hh.rel_err(seen["calls"][0], gW_ref) < 1e-5
        if kind == "post_accumulate_hook":
            assert Hh.rel_err(seen["calls"][-1], gW_ref) < 1e-5


def test_max_pooling_with_crystal_indices_that_do_not_start_at_zero():
    from crystalframer_amd import latticeformer
    dev = torch.device("cuda:0")
    sizes = torch.tensor([3, 1, 4, 2])
    x = torch.randn(10, 7, device=dev)
    batch = torch.repeat_interleave(torch.arange(4), sizes).to(dev) + 5
    got = latticeformer.max_pool(x, batch, sizes.to(dev))
    want = torch.stack([c.max(0).values for c in torch.split_with_sizes(x, sizes.tolist())])
    assert torch.equal(got, want)


def test_status_word_reports_a_box_cut_back_to_the_largest_half_width():
    """A Gaussian so wide that the box rule asks for more than 32 cells along an axis: the kernels sum the
    clamped box and say so in the status word of the workspace (0 for ordinary inputs)."""
    import crystalframer_amd as cf
    from crystalframer_amd import _lib
    dev = torch.device("cuda:0")
    P = Hh.make_problem(num_crystals=2, atoms_lo=1, atoms_hi=2, len_lo=2.0, len_hi=2.5, seed=5)
    g = lambda t: t.to(dtype=torch.float32, device=dev)

    def run(a):
        out = cf.RealEncodingWithFramedProjFuncCUDA.apply(
            g(a), g(P.rpos), None, g(P.tvecs), P.batch.to(dev), P.edges.to(dev), 0, 14.0, 1.0, None, None, None, None,
            None, None, None, 0, 4.0, 0, 1.0, 1.0, g(P.rvlen), -3.5)
        torch.cuda.synchronize()
        return out[0]

    _lib.read_status(dev, reset=True)
    z = run(P.a)
    assert torch.isfinite(z).all() and _lib.read_status(dev) == 0
    z = run(torch.full_like(P.a, -1e-3))        # sigma = 22 angstrom in 2 angstrom cells: half-width ~ 39
    assert torch.isfinite(z).all() and _lib.read_status(dev, reset=True) == 1
    assert _lib.read_status(dev) == 0
