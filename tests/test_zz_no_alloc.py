"""The entry point that allocates nothing (cfh_framed_pe_forward_static: scratch in a file-scope device array
of the library) against cfh_framed_pe_forward with a caller-provided workspace, through the C ABI: same
kernels on the same numbers, so z, psi, d2min and the kept histograms must be equal bit for bit.  Two calls
in a row, the second on a smaller input (the array keeps the first call's contents)."""
import ctypes

import pytest
import torch

import helpers as Hh

pytestmark = pytest.mark.gpu


def _call(lib, _lib, cf, P, static, dev):
    g = lambda t: None if t is None else t.to(dtype=torch.float32, device=dev).contiguous()
    N, E, B = P.N, P.E, P.tvecs.shape[0]
    a, rpos, tv, rv = g(P.a), g(P.rpos), g(P.tvecs), g(P.rvlen)
    batch, edges = P.batch.to(dev), P.edges.to(dev).contiguous()
    e_start, order = cf.cuda_funcs.edge_schedule(edges, N)
    Wd = g(P.W_k[0])
    Wa = [g(w[0]) for w in P.W_ax]
    frames = torch.stack([g(f) for f in P.frames], 0).contiguous()
    p = cf.cuda_funcs._params(Hh.H, Hh.DH, 64, 64, 0, Hh.DIST_MAX, 1.0, 4.0, 0.75, 1.25, -3.5)
    z = torch.full((E, Hh.H), float("nan"), device=dev)
    psi = torch.full((E, Hh.H, Hh.DH), float("nan"), device=dev)
    d2 = torch.full((E, Hh.H), float("nan"), device=dev)
    shat = torch.full((E, Hh.H, 4, 64), float("nan"), device=dev)
    st = _lib.current_stream_ptr(dev)
    head = (ctypes.byref(p), _lib.ptr(a), _lib.ptr(rpos), _lib.ptr(tv), _lib.ptr(rv), _lib.ptr(batch), _lib.ptr(edges),
            _lib.ptr(e_start), _lib.ptr(order), _lib.ptr(Wd), _lib.ptr(Wa[0]), _lib.ptr(Wa[1]), _lib.ptr(Wa[2]),
            _lib.ptr(frames), N, E, B, _lib.ptr(z), _lib.ptr(psi), _lib.ptr(d2), _lib.ptr(shat))
    if static:
        rc = lib.cfh_framed_pe_forward_static(*head, st)
        _lib.check(rc, "cfh_framed_pe_forward_static")
    else:
        ws = torch.empty(lib.cfh_workspace_bytes(ctypes.byref(p), N, E), dtype=torch.uint8, device=dev)
        rc = lib.cfh_framed_pe_forward(*head, _lib.ptr(ws), ws.numel(), st)
        _lib.check(rc, "cfh_framed_pe_forward")
    torch.cuda.synchronize()
    return z, psi, d2, shat


def test_static_scratch_forward_equals_workspace_forward_twice_second_smaller():
    import crystalframer_amd as cf
    from crystalframer_amd import _lib
    lib = _lib.load()
    dev = torch.device("cuda:0")
    big = Hh.make_problem(num_crystals=24, atoms_hi=9, seed=71)
    small = Hh.make_problem(num_crystals=3, atoms_hi=3, seed=72)
    with torch.cuda.device(dev):
        for P in (big, small):
            got = _call(lib, _lib, cf, P, True, dev)
            want = _call(lib, _lib, cf, P, False, dev)
            for x, y in zip(got, want):
                assert torch.isfinite(x).all()
                assert torch.equal(x, y)


def test_static_scratch_forward_rejects_what_it_cannot_hold():
    import crystalframer_amd as cf
    from crystalframer_amd import _lib
    lib = _lib.load()
    p = cf.cuda_funcs._params(Hh.H, Hh.DH, 64, 64, 0, Hh.DIST_MAX, 1.0, 4.0, 1.0, 1.0, -3.5)
    too_many = 65536 // Hh.H + 1
    rc = lib.cfh_framed_pe_forward_static(ctypes.byref(p), *([None] * 13), too_many, 1, 1, None, None, None, None, None)
    assert rc == -1 and b"static scratch" in lib.cfh_last_error()


def test_static_scratch_forward_under_graph_capture_and_with_timing_on():
    """The advertised caller: the entry point recorded into a HIP graph (a capture forbids allocations) with the
    library's timing diagnostics switched on (they create events, which this entry point must therefore skip);
    three replays with eager work in between, each equal to the workspace variant; device memory in use does not
    change over the calls."""
    import crystalframer_amd as cf
    from crystalframer_amd import _lib
    lib = _lib.load()
    dev = torch.device("cuda:0")
    P = Hh.make_problem(num_crystals=10, atoms_hi=7, seed=73)
    want = _call(lib, _lib, cf, P, False, dev)
    g = lambda t: t.to(dtype=torch.float32, device=dev).contiguous()
    N, E, B = P.N, P.E, P.tvecs.shape[0]
    a, rpos, tv, rv = g(P.a), g(P.rpos), g(P.tvecs), g(P.rvlen)
    batch, edges = P.batch.to(dev), P.edges.to(dev).contiguous()
    e_start, order = cf.cuda_funcs.edge_schedule(edges, N)
    Wd = g(P.W_k[0])
    Wa = [g(w[0]) for w in P.W_ax]
    frames = torch.stack([g(f) for f in P.frames], 0).contiguous()
    p = cf.cuda_funcs._params(Hh.H, Hh.DH, 64, 64, 0, Hh.DIST_MAX, 1.0, 4.0, 0.75, 1.25, -3.5)
    z = torch.zeros((E, Hh.H), device=dev)
    psi = torch.zeros((E, Hh.H, Hh.DH), device=dev)
    d2 = torch.zeros((E, Hh.H), device=dev)
    shat = torch.zeros((E, Hh.H, 4, 64), device=dev)

    def call():
        rc = lib.cfh_framed_pe_forward_static(
            ctypes.byref(p), _lib.ptr(a), _lib.ptr(rpos), _lib.ptr(tv), _lib.ptr(rv), _lib.ptr(batch), _lib.ptr(edges),
            _lib.ptr(e_start), _lib.ptr(order), _lib.ptr(Wd), _lib.ptr(Wa[0]), _lib.ptr(Wa[1]), _lib.ptr(Wa[2]),
            _lib.ptr(frames), N, E, B, _lib.ptr(z), _lib.ptr(psi), _lib.ptr(d2), _lib.ptr(shat),
            _lib.current_stream_ptr(dev))
        _lib.check(rc, "cfh_framed_pe_forward_static")

    _lib.read_kernel_timing("framed_pe_forward")
    _lib.kernel_timing(True)
    try:
        with torch.cuda.device(dev):
            side = torch.cuda.Stream()
            side.wait_stream(torch.cuda.current_stream())
            with torch.cuda.stream(side):
                call()                                   # first call on the device: symbol look-up
            torch.cuda.current_stream().wait_stream(side)
            torch.cuda.synchronize()
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph, stream=side):
                call()
            for rep in range(3):
                for t in (z, psi, d2, shat):
                    t.fill_(float("nan"))                # eager work between the replays
                torch.cuda.synchronize()
                graph.replay()
                torch.cuda.synchronize()
                for x, y in zip((z, psi, d2, shat), want):
                    assert torch.equal(x, y), rep
            free0 = torch.cuda.mem_get_info(dev)[0]
            call()
            torch.cuda.synchronize()
            assert torch.cuda.mem_get_info(dev)[0] == free0
    finally:
        _lib.kernel_timing(False)
    total, count = _lib.read_kernel_timing("framed_pe_forward")
    assert count == 0          # no events were created for the static calls
