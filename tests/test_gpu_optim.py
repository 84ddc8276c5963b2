"""The library's batched AdamW against torch.optim.AdamW (the optimizer of the reference's trainer,
models/regression.py:298-301): same parameters after several steps, relative tolerance 1e-6 of the tensor's largest
magnitude per step count (float32 rounding of the same formula in a different order)."""
import pytest
import torch

pytestmark = pytest.mark.gpu


def _params(dev, seed=0):
    gen = torch.Generator().manual_seed(seed)
    shapes = [(128, 128), (384, 128), (1,), (3,), (7, 5), (1023,), (1025,), (8, 16, 64), (98, 128), (4097,)]
    base = torch.randn(3 * 64 * 33, generator=gen)
    ps = [torch.randn(*s, generator=gen) for s in shapes]
    return ps, base


def _twin(dev, seed=0):
    """Leaf parameters; two of them views of one storage at an offset that is not a multiple of 16 bytes."""
    ps, base = _params(dev, seed)
    out = [torch.nn.Parameter(p.to(dev)) for p in ps]
    stack = base.to(dev)
    a = torch.nn.Parameter(stack[1:1 + 64 * 33].view(64, 33))
    b = torch.nn.Parameter(stack[1 + 64 * 33:1 + 2 * 64 * 33].view(64, 33))
    frozen = torch.nn.Parameter(torch.ones(5, device=dev), requires_grad=False)
    return out + [a, b, frozen]


def _grads(params, step, seed=100):
    gen = torch.Generator().manual_seed(seed + step)
    for k, p in enumerate(params):
        if not p.requires_grad:
            continue
        if k == 3 and step == 1:
            p.grad = None          # a parameter without a gradient in one step is left alone, as torch does
            continue
        p.grad = (torch.randn(p.shape, generator=gen) * (0.1 + k)).to(p.device)


@pytest.mark.parametrize("betas", [(0.9, 0.98), (0.9, 0.999)])
@pytest.mark.parametrize("wd", [0.0, 1e-2])
def test_adamw_matches_torch(wd, betas):
    """(0.9, 0.999), the default of both optimizers: 1 - beta2^t cancels in float32 during the first steps, so the
    kernel makes the bias corrections in double, as the framework does on the host."""
    from crystalframer_amd import optim
    dev = torch.device("cuda:0")
    mine, ref = _twin(dev), _twin(dev)
    o1 = optim.AdamW(mine, lr=3e-3, betas=betas, eps=1e-8, weight_decay=wd)
    o2 = torch.optim.AdamW(ref, lr=3e-3, betas=betas, eps=1e-8, weight_decay=wd)
    for step in range(6):
        _grads(mine, step); _grads(ref, step)
        before = mine[3].detach().clone()
        o1.step(); o2.step()
        if step == 1:
            assert torch.equal(mine[3], before)
        for k, (a, b) in enumerate(zip(mine, ref)):
            if k == 3 and step >= 1:
                continue      # torch counts steps per parameter, the library per group: they differ after a skipped step
            err = (a - b).abs().max().item() / max(b.abs().max().item(), 1e-30)
            assert err < 2e-6 * (step + 1), (k, step, err)
    assert torch.equal(mine[-1], torch.ones(5, device=dev))
    # the moments are visible under torch's names and survive a round trip through state_dict
    sd = o1.state_dict()
    o3 = optim.AdamW(mine, lr=3e-3, betas=betas, eps=1e-8, weight_decay=wd)
    o3.load_state_dict(sd)
    assert torch.equal(o3.state[mine[0]]["exp_avg"], o1.state[mine[0]]["exp_avg"])
    assert int(o3.state[mine[0]]["step"]) == 6


def test_adamw_in_a_captured_graph_keeps_counting():
    from crystalframer_amd import optim
    dev = torch.device("cuda:0")
    mine, ref = _twin(dev, 3), _twin(dev, 3)
    gbuf = [torch.zeros_like(p) for p in mine]
    for p, g in zip(mine, gbuf):
        if p.requires_grad:
            p.grad = g
    o1 = optim.AdamW(mine, lr=1e-2, betas=(0.8, 0.9), weight_decay=1e-3)
    o2 = torch.optim.AdamW(ref, lr=1e-2, betas=(0.8, 0.9), weight_decay=1e-3)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        o1.step()                                  # allocates the state outside the capture
    torch.cuda.current_stream().wait_stream(side)
    for p in ref:
        if p.requires_grad:
            p.grad = torch.zeros_like(p)
    o2.step()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        o1.step()
    for step in range(4):
        gen = torch.Generator().manual_seed(50 + step)
        for p, g, r in zip(mine, gbuf, ref):
            if p.requires_grad:
                val = torch.randn(p.shape, generator=gen).to(dev)
                g.copy_(val)
                r.grad = val.clone()
        graph.replay()
        torch.cuda.synchronize()
        o2.step()
        for a, b in zip(mine, ref):
            err = (a - b).abs().max().item() / max(b.abs().max().item(), 1e-30)
            assert err < 2e-6 * (step + 2), (step, err)
