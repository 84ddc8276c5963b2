"""Parity of the HIP attention (softmax over the pairs of an atom, with logit and value biases) and
of the per-crystal mean against the float64 oracles, forward and backward, through the
autograd.Function boundary (which calls the C ABI).  float32 kernels vs float64 oracle: 2e-5 of the
largest magnitude forward, 5e-5 for gradients."""
import pytest
import torch

import helpers as Hh
from oracle import c_oracle as CO
from oracle import torch_oracle as TO

pytestmark = pytest.mark.gpu


def dev():
    return torch.device("cuda:0")


def f32(t):
    return t.to(dtype=torch.float32, device=dev())


def attention_case(P, seed, with_a=True, with_b=True, big_logits=False):
    g = torch.Generator().manual_seed(seed)
    z = torch.randn(P.E, Hh.H, generator=g, dtype=torch.float64) * (30.0 if big_logits else 1.0) if with_a else None
    psi = torch.randn(P.E, Hh.H, Hh.DH, generator=g, dtype=torch.float64) if with_b else None
    gout = torch.randn(P.N, Hh.H, Hh.DH, generator=g, dtype=torch.float64)
    return z, psi, gout


def run_both(P, z, psi, gout):
    import crystalframer_amd as cf
    leaves64 = [t.double().clone().requires_grad_(True) if t is not None else None for t in (P.q, P.k, P.v, z, psi)]
    out64, prob64 = TO.softmax_attention(*leaves64, P.batch, P.edges)
    (out64 * gout).sum().backward()
    leaves = [f32(t).requires_grad_(True) if t is not None else None for t in (P.q, P.k, P.v, z, psi)]
    out = cf.FusedDotProductAttentionCUDA.apply(*leaves, P.batch.to(dev()), P.edges.to(dev()))
    (out * f32(gout)).sum().backward()
    return out64, leaves64, out, leaves


@pytest.mark.parametrize("with_a,with_b", [(True, True), (True, False), (False, False)])
def test_attention_forward_backward(with_a, with_b):
    P = Hh.make_problem(num_crystals=7, atoms_hi=9, seed=71)
    z, psi, gout = attention_case(P, 5, with_a, with_b)
    out64, leaves64, out, leaves = run_both(P, z, psi, gout)
    assert Hh.rel_err(out.cpu().double(), out64.detach()) < 2e-5
    for l32, l64, name in zip(leaves, leaves64, "q k v a b".split()):
        if l64 is None:
            continue
        assert Hh.rel_err(l32.grad.cpu().double(), l64.grad) < 5e-5, name


def test_attention_matches_c_oracle_and_saves_probabilities():
    import crystalframer_amd as cf
    from crystalframer_amd import _lib
    P = Hh.make_problem(num_crystals=5, atoms_hi=6, seed=72)
    z, psi, gout = attention_case(P, 6)
    oc, pc = CO.dpa_forward(P.q, P.k, P.v, z, psi, P.edges, "f64")
    # straight through the C ABI
    lib = _lib.load()
    q, k, v, a, b = (f32(t).contiguous() for t in (P.q, P.k, P.v, z, psi))
    edges = P.edges.to(dev()).contiguous()
    e_start, _ = cf.cuda_funcs.edge_schedule(edges, P.N)
    out = torch.empty_like(v)
    prob = torch.empty(P.E, Hh.H, device=dev())
    rc = lib.cfh_fused_dpa_forward(_lib.ptr(q), _lib.ptr(k), _lib.ptr(v), _lib.ptr(a), _lib.ptr(b), _lib.ptr(edges),
                                   _lib.ptr(e_start), P.N, Hh.H, Hh.DH, P.E, _lib.ptr(prob), _lib.ptr(out),
                                   _lib.current_stream_ptr(dev()))
    assert rc == 0
    assert Hh.rel_err(out.cpu().double(), oc) < 2e-5
    assert Hh.rel_err(prob.cpu().double(), pc) < 2e-5
    rowsum = torch.zeros(P.N, Hh.H, device=dev()).index_add_(0, edges[0], prob)
    assert (rowsum - 1).abs().max() < 1e-5


def test_attention_large_logits_and_long_rows():
    """Rows longer than the 4 pairs in flight and logits of magnitude ~100: the running-maximum
    softmax must neither overflow nor lose the small terms."""
    P = Hh.make_problem(num_crystals=3, atoms_lo=17, atoms_hi=23, seed=73)
    z, psi, gout = attention_case(P, 7, big_logits=True)
    out64, leaves64, out, leaves = run_both(P, z, psi, gout)
    assert torch.isfinite(out).all()
    assert Hh.rel_err(out.cpu().double(), out64.detach()) < 2e-5
    for l32, l64 in zip(leaves, leaves64):
        assert Hh.rel_err(l32.grad.cpu().double(), l64.grad) < 5e-5


def test_attention_single_atom_crystals_and_empty():
    import crystalframer_amd as cf
    P = Hh.make_problem(num_crystals=4, atoms_lo=1, atoms_hi=1, seed=74)
    z, psi, gout = attention_case(P, 8)
    out64, leaves64, out, leaves = run_both(P, z, psi, gout)
    # one pair per atom: probability 1, out = v + b
    assert Hh.rel_err(out.cpu().double(), (P.v.double() + psi)) < 1e-6
    assert leaves[3].grad.abs().max() < 1e-5          # p (gp - D) cancels up to rounding
    q = torch.zeros(0, Hh.H, Hh.DH, device=dev())
    out = cf.FusedDotProductAttentionCUDA.apply(q, q, q, torch.zeros(0, Hh.H, device=dev()),
                                                torch.zeros(0, Hh.H, Hh.DH, device=dev()),
                                                torch.zeros(0, dtype=torch.long, device=dev()),
                                                torch.zeros(2, 0, dtype=torch.long, device=dev()))
    assert out.shape == (0, Hh.H, Hh.DH)


def test_attention_backward_rejects_incomplete_pair_blocks():
    import crystalframer_amd as cf
    P = Hh.make_problem(num_crystals=3, atoms_lo=3, atoms_hi=4, seed=75)
    keep = torch.ones(P.E, dtype=torch.bool)
    keep[1] = False                                   # drop one pair: no longer n x n
    edges = P.edges[:, keep].to(dev()).contiguous()
    z, psi, gout = attention_case(P, 9)
    leaves = [f32(t).requires_grad_(True) for t in (P.q, P.k, P.v, z[keep], psi[keep])]
    out = cf.FusedDotProductAttentionCUDA.apply(*leaves, P.batch.to(dev()), edges)
    # the forward needs no such layout and still matches
    o64, _ = TO.softmax_attention(P.q.double(), P.k.double(), P.v.double(), z[keep], psi[keep], P.batch, P.edges[:, keep])
    assert Hh.rel_err(out.detach().cpu().double(), o64) < 2e-5
    with pytest.raises(ValueError, match="complete"):
        out.sum().backward()


def test_attention_full_batch_properties():
    """Batch of 256 crystals: rows sum to one, out is a convex combination (bounded by the values),
    the value gradients sum to the upstream gradient, and a constant shift of a row's logits changes
    nothing."""
    import crystalframer_amd as cf
    from crystalframer_amd import geometry, synthetic
    cb = synthetic.make_config("C3", seed=5).to(dev())
    geo = geometry.crystal_geometry(cb.pos, cb.batch, cb.trans_vec, cb.sizes)
    N, E, H, D = cb.pos.shape[0], geo.num_edges, 8, 16
    g = torch.Generator(device="cpu").manual_seed(11)
    q = (torch.randn(N, H, D, generator=g) / 4).to(dev())
    k = torch.randn(N, H, D, generator=g).to(dev())
    v = torch.randn(N, H, D, generator=g).to(dev()).requires_grad_(True)
    a = torch.randn(E, H, generator=g).to(dev())
    out = cf.FusedDotProductAttentionCUDA.apply(q, k, v, a, None, cb.batch, geo.edges)
    vmax = torch.zeros(N, H, D, device=dev()).scatter_reduce(0, geo.edges[0][:, None, None].expand(-1, H, D),
                                                             v.detach()[geo.edges[1]], reduce="amax", include_self=False)
    assert (out.detach() <= vmax + 1e-5).all()
    shift = torch.randn(N, H, generator=g).to(dev()) * 5
    out2 = cf.FusedDotProductAttentionCUDA.apply(q, k, v, a + shift[geo.edges[0]], None, cb.batch, geo.edges)
    assert (out2 - out).abs().max() < 2e-5
    go = torch.randn(N, H, D, generator=g).to(dev())
    (out * go).sum().backward()
    # sum_j gv_j = sum_i go_i within each crystal (probabilities of a row sum to one)
    per_crystal = lambda t: torch.zeros(cb.sizes.shape[0], H, D, device=dev()).index_add_(0, cb.batch, t)
    assert Hh.rel_err(per_crystal(v.grad).cpu(), per_crystal(go).cpu()) < 1e-5


def test_crystal_mean_forward_backward():
    import crystalframer_amd as cf
    sizes = torch.tensor([2, 1, 7, 4, 30])
    batch = torch.repeat_interleave(torch.arange(5), sizes)
    x64 = torch.randn(int(sizes.sum()), 128, dtype=torch.float64, requires_grad=True)
    ref = TO.crystal_mean(x64, batch, 5)
    gout = torch.randn(5, 128, dtype=torch.float64)
    (ref * gout).sum().backward()
    x = f32(x64.detach()).requires_grad_(True)
    out = cf.IrregularMeanCUDA.apply(x, batch.to(dev()), sizes.to(dev()))
    (out * f32(gout)).sum().backward()
    assert Hh.rel_err(out.detach().cpu().double(), ref.detach()) < 1e-6
    assert Hh.rel_err(x.grad.cpu().double(), x64.grad) < 1e-6
    # sizes derived from batch, odd channel count
    x3 = torch.randn(int(sizes.sum()), 5, device=dev())
    out3 = cf.IrregularMeanCUDA.apply(x3, batch.to(dev()), None)
    ref3 = TO.crystal_mean(x3.cpu().double(), batch, 5)
    assert Hh.rel_err(out3.cpu().double(), ref3) < 1e-6
    # rows of three 16-byte quads (the slices of a block do not fill it), a long crystal, an empty one
    sizes12 = torch.tensor([199, 0, 1, 64])
    batch12 = torch.repeat_interleave(torch.arange(4), sizes12)
    x12 = torch.randn(int(sizes12.sum()), 12, device=dev())
    out12 = cf.IrregularMeanCUDA.apply(x12, batch12.to(dev()), sizes12.to(dev()))
    ref12 = torch.stack([x12[batch12.to(dev()) == b].cpu().double().mean(0) if sizes12[b] > 0
                         else torch.zeros(12, dtype=torch.float64) for b in range(4)])
    assert Hh.rel_err(out12.cpu().double(), ref12) < 1e-6


def test_second_stream_fork_and_join_order_a_library_call():
    """Work put on the library's second stream between fork and join is ordered like work on the caller's."""
    import ctypes
    from crystalframer_amd import _lib
    lib = _lib.load()
    sizes = torch.tensor([3, 5, 1, 40])
    start = torch.nn.functional.pad(torch.cumsum(sizes, 0), (1, 0)).to(dev())
    x = torch.randn(int(sizes.sum()), 128, device=dev())
    out = torch.full((4, 128), float("nan"), device=dev())
    x2 = x * 2.0                                        # produced on the caller's stream before the fork
    cur = _lib.current_stream_ptr(dev())
    side, side2 = ctypes.c_void_p(), ctypes.c_void_p()
    _lib.check(lib.cfh_second_stream_fork(cur, ctypes.byref(side)), "fork")
    _lib.check(lib.cfh_second_stream_get(ctypes.byref(side2)), "get")
    assert side.value is not None and side.value == side2.value and side.value != (cur.value or 0)
    _lib.check(lib.cfh_crystal_mean_forward(_lib.ptr(x2), _lib.ptr(start), x.shape[0], 4, 128, _lib.ptr(out), side), "mean")
    _lib.check(lib.cfh_second_stream_join(cur), "join")
    res = out + 0.0                                     # consumer on the caller's stream after the join
    ref = torch.stack([x2[start[b]:start[b + 1]].mean(0) for b in range(4)])
    assert Hh.rel_err(res, ref) < 1e-6


@pytest.mark.parametrize("N,I,O,bias", [(2372, 128, 384, True), (2372, 512, 128, True), (2372, 98, 128, False),
                                        (37, 20, 50, True), (1, 16, 16, True), (0, 16, 32, True),
                                        # multiples of 64 take the kernel variant with 16-byte loads: few rows (wavefronts
                                        # of a workgroup without rows), rows that do not fill the last chunk
                                        (37, 64, 128, True), (5, 128, 64, True), (1001, 64, 64, False), (1, 64, 64, True)])
def test_linear_weight_and_bias_gradients(N, I, O, bias):
    """The library's weight/bias gradient kernel against float64 autograd of x W^T + b."""
    import crystalframer_amd as cf
    gen = torch.Generator().manual_seed(N + I + O)
    x64 = torch.randn(N, I, generator=gen, dtype=torch.float64, requires_grad=True)
    w64 = torch.randn(O, I, generator=gen, dtype=torch.float64, requires_grad=True)
    b64 = torch.randn(O, generator=gen, dtype=torch.float64, requires_grad=True) if bias else None
    gy = torch.randn(N, O, generator=gen, dtype=torch.float64)
    (torch.nn.functional.linear(x64, w64, b64) * gy).sum().backward()
    x = f32(x64.detach()).requires_grad_(True)
    w = f32(w64.detach()).requires_grad_(True)
    b = f32(b64.detach()).requires_grad_(True) if bias else None
    y = cf.cuda_funcs.linear(x, w, b)
    (y * f32(gy)).sum().backward()
    if N > 0:
        assert Hh.rel_err(y, torch.nn.functional.linear(x64, w64, b64)) < 1e-5
        assert Hh.rel_err(x.grad, x64.grad) < 1e-5
        assert Hh.rel_err(w.grad, w64.grad) < 1e-5
        if bias:
            assert Hh.rel_err(b.grad, b64.grad) < 1e-5
    else:
        assert float(w.grad.abs().max()) == 0.0 and float(b.grad.abs().max()) == 0.0


@pytest.mark.parametrize("N,H,normalised", [(2372, 8, True), (37, 8, False), (5, 2, True), (1, 16, True), (0, 8, True)])
def test_attention_inputs_split_scale_and_gaussian_coefficient(N, H, normalised):
    """q/k/v split + query scaling + Gaussian coefficient in one launch against the float64
    framework arithmetic (alpha = q.w, normalised, elu, affine), forward and gradients."""
    import math
    import crystalframer_amd as cf
    Dh, lb, beta, scale_real = 16, 0.5, 0.1, 1.4
    c1, c2 = beta / (1.0 - lb), -0.5 * scale_real ** -2
    gen = torch.Generator().manual_seed(100 + N + H)
    qkv64 = (torch.randn(N, 3 * H * Dh, generator=gen, dtype=torch.float64) * 3).requires_grad_(True)
    w64 = torch.randn(H * Dh, generator=gen, dtype=torch.float64, requires_grad=True)
    gs64 = torch.tensor([0.37, -0.8], dtype=torch.float64) if normalised else None
    q, k, v = (t.reshape(N, H, Dh) for t in qkv64.split(H * Dh, dim=1))
    alpha = (q * w64.view(1, H, Dh)).sum(-1)
    if normalised:
        alpha = (alpha + gs64[1]) * gs64[0]
    a64 = ((1.0 - lb) * torch.nn.functional.elu(alpha * c1) + 1.0) * c2
    qs64 = q / math.sqrt(Dh)
    g = [torch.randn(t.shape, generator=gen, dtype=torch.float64) for t in (qs64, k, v, a64)]
    sum((o * gi).sum() for o, gi in zip((qs64, k, v, a64), g)).backward()

    qkv = f32(qkv64.detach()).requires_grad_(True)
    w = f32(w64.detach()).requires_grad_(True)
    gs = f32(gs64) if normalised else None
    outs = cf.cuda_funcs.AttentionInputsHIP.apply(qkv, w, gs, H, c1, lb, c2, 1.0 / math.sqrt(Dh))
    assert [tuple(o.shape) for o in outs] == [(N, H, Dh)] * 3 + [(N, H)]
    sum((o * f32(gi)).sum() for o, gi in zip(outs, g)).backward()
    if N == 0:
        assert float(w.grad.abs().max()) == 0.0
        return
    for o, ref in zip(outs, (qs64, k, v, a64)):
        assert Hh.rel_err(o.detach(), ref.detach()) < 1e-6
    assert Hh.rel_err(qkv.grad, qkv64.grad) < 1e-6
    assert Hh.rel_err(w.grad, w64.grad) < 1e-5
    # only the value gradient given: the others count as zero
    qkv.grad = None
    outs = cf.cuda_funcs.AttentionInputsHIP.apply(qkv, w, gs, H, c1, lb, c2, 1.0 / math.sqrt(Dh))
    (outs[2] * f32(g[2])).sum().backward()
    expect = torch.cat([torch.zeros(N, 2 * H * Dh, dtype=torch.float64), g[2].reshape(N, -1)], dim=1)
    assert Hh.rel_err(qkv.grad, expect) < 1e-6
    assert Hh.rel_err(w.grad, w64.grad) < 1e-5           # a zero contribution was added to the existing .grad
    # a second full pass accumulates; the sum of the per-block partials is deferred to the end of the
    # pass for a leaf weight and made at once otherwise: same numbers
    outs = cf.cuda_funcs.AttentionInputsHIP.apply(qkv, w, gs, H, c1, lb, c2, 1.0 / math.sqrt(Dh))
    sum((o * f32(gi)).sum() for o, gi in zip(outs, g)).backward()
    assert Hh.rel_err(w.grad, 2 * w64.grad) < 1e-5
    w_mid = w * 1.0                                      # not a leaf
    outs = cf.cuda_funcs.AttentionInputsHIP.apply(qkv, w_mid, gs, H, c1, lb, c2, 1.0 / math.sqrt(Dh))
    gw_now, = torch.autograd.grad(sum((o * f32(gi)).sum() for o, gi in zip(outs, g)), [w_mid])
    assert Hh.rel_err(gw_now, w64.grad) < 1e-5
    outs = cf.cuda_funcs.AttentionInputsHIP.apply(qkv, w, gs, H, c1, lb, c2, 1.0 / math.sqrt(Dh))
    gw_leaf, = torch.autograd.grad(sum((o * f32(gi)).sum() for o, gi in zip(outs, g)), [w])
    assert Hh.rel_err(gw_leaf, w64.grad) < 1e-5
    assert Hh.rel_err(w.grad, 2 * w64.grad) < 1e-5       # autograd.grad leaves .grad alone


def test_weight_gradient_batch_job_without_weight_sums_columns():
    """A job of the batched weight-gradient launch with dW == NULL adds the column sums of dy to db,
    next to an ordinary job in the same launch."""
    import ctypes
    from crystalframer_amd import _lib
    lib = _lib.load()
    gen = torch.Generator().manual_seed(77)
    part = f32(torch.randn(297, 128, generator=gen, dtype=torch.float64))
    x = f32(torch.randn(150, 48, generator=gen, dtype=torch.float64))
    dy = f32(torch.randn(150, 40, generator=gen, dtype=torch.float64))
    out = torch.full((128,), 0.5, dtype=torch.float32, device=dev())
    dW = torch.zeros((40, 48), dtype=torch.float32, device=dev())
    db = torch.zeros((40,), dtype=torch.float32, device=dev())
    jobs = (_lib.CfhLinearGradJob * 2)()
    jobs[0].x, jobs[0].dy, jobs[0].dW, jobs[0].db = None, part.data_ptr(), None, out.data_ptr()
    jobs[0].N, jobs[0].I, jobs[0].O, jobs[0].ldx, jobs[0].ldy = 297, 1, 128, 1, 128
    jobs[1].x, jobs[1].dy, jobs[1].dW, jobs[1].db = x.data_ptr(), dy.data_ptr(), dW.data_ptr(), db.data_ptr()
    jobs[1].N, jobs[1].I, jobs[1].O, jobs[1].ldx, jobs[1].ldy = 150, 48, 40, 48, 40
    _lib.check(lib.cfh_linear_weight_bias_grad_batch(jobs, 2, None, 0, _lib.current_stream_ptr(part.device)), "batch")
    torch.cuda.synchronize()
    assert Hh.rel_err(out, 0.5 + part.double().sum(0)) < 1e-5
    assert Hh.rel_err(dW, dy.double().t() @ x.double()) < 1e-5
    assert Hh.rel_err(db, dy.double().sum(0)) < 1e-5
    # neither output given: refused
    jobs[0].db = None
    assert lib.cfh_linear_weight_bias_grad_batch(jobs, 1, None, 0, _lib.current_stream_ptr(part.device)) != 0


def test_weight_gradient_batch_sums_in_a_fixed_order_with_scratch():
    """With scratch the batched weight-gradient launch adds the row slices of every tile in a fixed order: the same
    bits on every run, the values those of the float64 products, accumulated into what dW and db held.  Jobs of both
    kernel variants (16-byte loads: O and I multiples of 64; scalar loads with ragged edges), a bias-only job, a job
    with a single slice (16 rows), and a second call with fewer jobs on the same scratch."""
    from crystalframer_amd import _lib
    lib = _lib.load()
    gen = torch.Generator().manual_seed(78)
    rnd = lambda *s: f32(torch.randn(*s, generator=gen, dtype=torch.float64))
    shapes = [(3001, 128, 128, True), (3001, 128, 384, True), (1777, 48, 40, True), (16, 64, 64, True), (2500, 1, 128, False),
              (2222, 100, 70, False)]
    ops = []
    for N, I, O, has_b in shapes:
        x, dy = rnd(N, I), rnd(N, O)
        ops.append((x, dy, rnd(O, I) if I > 1 else None, rnd(O)))

    def run(n_jobs):
        outs = []
        jobs = (_lib.CfhLinearGradJob * n_jobs)()
        for J, (x, dy, w0, b0) in zip(jobs, ops):
            dW = None if w0 is None else w0.clone()
            db = b0.clone()
            J.x, J.dy = (None if w0 is None else x.data_ptr()), dy.data_ptr()
            J.dW, J.db = (None if dW is None else dW.data_ptr()), db.data_ptr()
            J.N, J.I, J.O, J.ldx, J.ldy = x.shape[0], x.shape[1], dy.shape[1], x.shape[1], dy.shape[1]
            outs.append((dW, db))
        need = lib.cfh_linear_weight_bias_grad_batch_workspace_bytes(jobs, n_jobs)
        assert need > 0
        ws = _lib.wgrad_scratch(dev(), _lib.current_stream_ptr(dev()), need)
        _lib.check(lib.cfh_linear_weight_bias_grad_batch(jobs, n_jobs, _lib.ptr(ws), ws.numel(),
                                                         _lib.current_stream_ptr(dev())), "batch")
        torch.cuda.synchronize()
        # too small a scratch is refused
        assert lib.cfh_linear_weight_bias_grad_batch(jobs, n_jobs, _lib.ptr(ws), 256,
                                                     _lib.current_stream_ptr(dev())) != 0
        return outs

    first = run(len(ops))
    for (dW, db), (x, dy, w0, b0) in zip(first, ops):
        if dW is not None:
            assert Hh.rel_err(dW, w0.double() + dy.double().t() @ x.double()) < 1e-5
        assert Hh.rel_err(db, b0.double() + dy.double().sum(0)) < 1e-5
    for _ in range(3):
        again = run(len(ops))
        for (dW, db), (dW2, db2) in zip(first, again):
            assert dW is None or torch.equal(dW, dW2)
            assert torch.equal(db, db2)
    # fewer jobs: other slice counts per tile, the same scratch
    fewer = run(2)
    for (dW, db), (x, dy, w0, b0) in zip(fewer, ops):
        assert Hh.rel_err(dW, w0.double() + dy.double().t() @ x.double()) < 1e-5
        assert Hh.rel_err(db, b0.double() + dy.double().sum(0)) < 1e-5
    assert all(torch.equal(a[0], b[0]) and torch.equal(a[1], b[1]) for a, b in zip(fewer, run(2)))

    # two jobs that add to the same dW and db (a weight used twice in one pass): both arrive, in the jobs' order
    def shared():
        x, dy, w0, b0 = ops[0]
        x2, dy2 = ops[1][0], ops[1][1][:, :128].contiguous()
        dW, db = w0.clone(), b0.clone()
        jobs = (_lib.CfhLinearGradJob * 2)()
        for J, (xx, yy) in zip(jobs, ((x, dy), (x2, dy2))):
            J.x, J.dy, J.dW, J.db = xx.data_ptr(), yy.data_ptr(), dW.data_ptr(), db.data_ptr()
            J.N, J.I, J.O, J.ldx, J.ldy = xx.shape[0], 128, 128, 128, 128
        ws = _lib.wgrad_scratch(dev(), _lib.current_stream_ptr(dev()),
                                lib.cfh_linear_weight_bias_grad_batch_workspace_bytes(jobs, 2))
        _lib.check(lib.cfh_linear_weight_bias_grad_batch(jobs, 2, _lib.ptr(ws), ws.numel(),
                                                         _lib.current_stream_ptr(dev())), "batch")
        torch.cuda.synchronize()
        ref = w0.double() + dy.double().t() @ x.double() + dy2.double().t() @ x2.double()
        assert Hh.rel_err(dW, ref) < 1e-5
        assert Hh.rel_err(db, b0.double() + dy.double().sum(0) + dy2.double().sum(0)) < 1e-5
        return dW, db
    s1, s2 = shared(), shared()
    assert torch.equal(s1[0], s2[0]) and torch.equal(s1[1], s2[1])


def test_linear_deferred_gradients_stacked_accumulated_and_nonleaf():
    """The deferred weight-gradient launch: several layers in one backward pass (one of them with three
    stacked weights sharing a bias), a second pass accumulating into existing .grad, a weight that is
    not a leaf (gradient needed before the pass ends), and torch.autograd.grad instead of backward."""
    import crystalframer_amd as cf
    lin = cf.cuda_funcs.linear
    gen = torch.Generator().manual_seed(9)
    N = 301
    mk = lambda *shape: torch.randn(*shape, generator=gen, dtype=torch.float64)
    x64 = mk(N, 48).requires_grad_(True)
    ws64 = [mk(32, 48).requires_grad_(True), mk(16, 48).requires_grad_(True), mk(64, 48).requires_grad_(True)]
    b64 = mk(112).requires_grad_(True)
    w2_64 = mk(40, 112).requires_grad_(True)
    b2_64 = mk(40).requires_grad_(True)
    scale64 = torch.tensor(0.7, dtype=torch.float64, requires_grad=True)
    leaves64 = [x64, *ws64, b64, w2_64, b2_64, scale64]

    def net(x, ws, b, w2, b2, scale, linear, cat):
        h = torch.tanh(linear(x, cat(ws), b))
        h = linear(h, w2 * scale, b2)              # a weight that is not a leaf
        return h.square().sum()

    ref = net(x64, ws64, b64, w2_64, b2_64, scale64, torch.nn.functional.linear, lambda ws: torch.cat(ws, 0))
    ref.backward()
    leaves = [f32(t.detach()).requires_grad_(True) for t in leaves64]
    x, w0, w1, w2s, b, w2, b2, scale = leaves

    def run():
        return net(x, [w0, w1, w2s], b, w2, b2, scale, lambda xx, ww, bb: lin(xx, ww, bb), lambda ws: tuple(ws))

    run().backward()
    for t32, t64 in zip(leaves, leaves64):
        assert Hh.rel_err(t32.grad, t64.grad) < 2e-5
    # second pass: gradients accumulate into the existing .grad tensors
    run().backward()
    for t32, t64 in zip(leaves, leaves64):
        assert Hh.rel_err(t32.grad, 2 * t64.grad) < 2e-5
    # autograd.grad returns complete gradients and leaves .grad alone
    before = w0.grad.clone()
    g = torch.autograd.grad(run(), [w0, b, w2])
    assert Hh.rel_err(g[0], ws64[0].grad) < 2e-5 and Hh.rel_err(g[1], b64.grad) < 2e-5 and Hh.rel_err(g[2], w2_64.grad) < 2e-5
    assert torch.equal(w0.grad, before)
    # deferral switched off gives the same numbers
    KM = cf.KernelManager
    KM.DEFER_WEIGHT_GRADS = False
    try:
        for t in leaves:
            t.grad = None
        run().backward()
    finally:
        KM.DEFER_WEIGHT_GRADS = True
    for t32, t64 in zip(leaves, leaves64):
        assert Hh.rel_err(t32.grad, t64.grad) < 2e-5


@pytest.mark.parametrize("M,I,O,bias,relu", [(256, 128, 128, True, True), (256, 128, 1, True, False), (37, 48, 20, False, False),
                                             (512, 64, 96, True, True), (1, 16, 16, True, False)])
def test_few_row_projection_kernels(M, I, O, bias, relu):
    """Projections with few rows take the library's own forward / input-gradient kernels: against
    float64 autograd of relu(x W^T + b)."""
    import crystalframer_amd as cf
    gen = torch.Generator().manual_seed(M + I + O)
    x64 = torch.randn(M, I, generator=gen, dtype=torch.float64, requires_grad=True)
    w64 = torch.randn(O, I, generator=gen, dtype=torch.float64, requires_grad=True)
    b64 = torch.randn(O, generator=gen, dtype=torch.float64, requires_grad=True) if bias else None
    gy = torch.randn(M, O, generator=gen, dtype=torch.float64)
    y64 = torch.nn.functional.linear(x64, w64, b64)
    if relu:
        y64 = torch.relu(y64)
    (y64 * gy).sum().backward()
    x = f32(x64.detach()).requires_grad_(True)
    w = f32(w64.detach()).requires_grad_(True)
    b = f32(b64.detach()).requires_grad_(True) if bias else None
    events = []
    cf.KernelManager.EVENT_LOG = events
    try:
        y = cf.cuda_funcs.linear(x, w, b, relu=relu)
        (y * f32(gy)).sum().backward()
    finally:
        cf.KernelManager.EVENT_LOG = None
    names = {e[0] for e in events}
    assert "small_linear_forward" in names                      # the library kernels were the ones that ran
    assert "small_linear_dx" in names                           # few output features take the plain-loop kernel
    assert Hh.rel_err(y, y64) < 1e-5
    assert Hh.rel_err(x.grad, x64.grad) < 1e-5
    assert Hh.rel_err(w.grad, w64.grad) < 1e-5
    if bias:
        assert Hh.rel_err(b.grad, b64.grad) < 1e-5


@pytest.mark.parametrize("N,has_next,normalised,with_bias", [(301, True, True, True), (16, True, False, False),
                                                              (77, False, False, True), (0, True, True, True)])
def test_layer_bridge_matches_framework_chain(N, has_next, normalised, with_bias):
    """Output projection + residual, feed-forward block + residual, next layer's input projection and
    attention inputs in one launch, against float64 autograd of the same chain; the backward pass
    (framework GEMMs + deferred weight gradients) gives every gradient, also when accumulated into
    existing .grad tensors by a second pass."""
    import math
    import crystalframer_amd as cf
    D, F, H, Dh, lb, beta, scale_real = 128, 256, 8, 16, 0.5, 0.1, 1.4
    c1, c2 = beta / (1.0 - lb), -0.5 * scale_real ** -2
    gen = torch.Generator().manual_seed(300 + N)
    mk = lambda *shape, s=1.0: torch.randn(*shape, generator=gen, dtype=torch.float64) * s
    t64 = dict(attn=mk(N, D), xres=mk(N, D), Wo=mk(D, D, s=D ** -0.5), W1=mk(F, D, s=D ** -0.5), W2=mk(D, F, s=F ** -0.5),
               Wq=mk(D, D, s=D ** -0.5), Wk=mk(D, D, s=D ** -0.5), Wv=mk(D, D, s=D ** -0.5), lw=mk(D, s=0.25))
    if with_bias:
        t64.update(bo=mk(D), b1=mk(F), b2=mk(D), bin=mk(3 * D))
    for t in t64.values():
        t.requires_grad_(True)
    gs64 = torch.tensor([0.37, -0.8], dtype=torch.float64) if normalised else None

    def chain(t, lin, relu, gs):
        x1 = t["xres"] + lin(t["attn"], t["Wo"], t.get("bo"))
        hh = relu(lin(x1, t["W1"], t.get("b1")))
        x2 = x1 + lin(hh, t["W2"], t.get("b2"))
        if not has_next:
            return (x2,)
        qkv = lin(x2, torch.cat([t["Wq"], t["Wk"], t["Wv"]], 0), t.get("bin"))
        q, k, v = (p.reshape(N, H, Dh) for p in qkv.split(D, dim=1))
        alpha = (q * t["lw"].view(1, H, Dh)).sum(-1)
        if gs is not None:
            alpha = (alpha + gs[1]) * gs[0]
        a = ((1.0 - lb) * torch.nn.functional.elu(alpha * c1) + 1.0) * c2
        return x2, q / math.sqrt(Dh), k, v, a

    ref = chain(t64, torch.nn.functional.linear, torch.relu, gs64)
    g = [torch.randn(o.shape, generator=gen, dtype=torch.float64) for o in ref]
    sum((o * gi).sum() for o, gi in zip(ref, g)).backward()

    t32 = {n: f32(t.detach()).requires_grad_(True) for n, t in t64.items()}
    gs = f32(gs64) if normalised else None

    def run():
        extra = (t32["Wq"], t32["Wk"], t32["Wv"]) if has_next else ()
        return cf.cuda_funcs.LayerBridgeHIP.apply(
            t32["attn"], t32["xres"], t32["Wo"], t32.get("bo"), t32["W1"], t32.get("b1"), t32["W2"], t32.get("b2"),
            None, t32.get("bin") if has_next else None, t32["lw"] if has_next else None, gs if has_next else None,
            H, c1, lb, c2, 1.0 / math.sqrt(Dh), *extra)

    outs = run()
    assert len(outs) == len(ref)
    for o, r in zip(outs, ref):
        assert o.shape == r.shape
        if N:
            assert Hh.rel_err(o.detach(), r.detach()) < 2e-6
    sum((o * f32(gi)).sum() for o, gi in zip(outs, g)).backward()
    used = [n for n in t64 if has_next or n not in ("Wq", "Wk", "Wv", "lw", "bin")]
    for n in used:
        if N == 0:
            assert t32[n].grad is None or float(t32[n].grad.abs().sum()) == 0.0
        else:
            assert Hh.rel_err(t32[n].grad, t64[n].grad) < 2e-5, n
    if N == 0:
        return
    outs = run()                                         # second pass: accumulation
    sum((o * f32(gi)).sum() for o, gi in zip(outs, g)).backward()
    for n in used:
        assert Hh.rel_err(t32[n].grad, 2 * t64[n].grad) < 2e-5, n
    # only the layer output is used downstream
    for t in t32.values():
        t.grad = None
    (run()[0] * f32(g[0])).sum().backward()
    assert t32["attn"].grad is not None and t32["W2"].grad is not None
    # the input gradients by framework GEMMs instead of the one launch: same numbers
    LB = cf.cuda_funcs.LayerBridgeHIP
    LB.FUSED_BACKWARD = False
    try:
        for t in t32.values():
            t.grad = None
        outs = run()
        sum((o * f32(gi)).sum() for o, gi in zip(outs, g)).backward()
    finally:
        LB.FUSED_BACKWARD = True
    for n in used:
        assert Hh.rel_err(t32[n].grad, t64[n].grad) < 2e-5, n
    # weight gradients made at once instead of at the end of the pass: same numbers
    KM = cf.KernelManager
    KM.DEFER_WEIGHT_GRADS = False
    try:
        for t in t32.values():
            t.grad = None
        outs = run()
        sum((o * f32(gi)).sum() for o, gi in zip(outs, g)).backward()
    finally:
        KM.DEFER_WEIGHT_GRADS = True
    for n in used:
        assert Hh.rel_err(t32[n].grad, t64[n].grad) < 2e-5, n
