#!/usr/bin/env python3
"""Benchmark of the periodic-attention hot path on one MI355X.

One "step" is one training step (forward, MSE loss, backward, AdamW update) of the 4-layer
CrystalFramer max-frame model over one batch of 256 synthetic crystals that is already resident in
HBM (configuration C3: the 4-layer max-frame model at batch 256; fp32, random-init weights).  Prints ONE JSON line with
crystals/s, the roofline figures of the dominant kernel measured with HIP events inside the library,
the other large configurations (C2, C4, C5) timed the same way, and the CPU baseline (the PyTorch restatement of
the reference's pure-PyTorch formulation, timed on the host cores on a bounded sample of the same batch).

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-cpu-baseline] [--no-other-configs]
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

# algorithmic work per unique lattice-pair term (reference semantics, windows 9 / 33 bins):
# geometry 23 flop, weight 3 flop + 1 exp, |d| and 1/|d|, window set-up 3 flop each,
# forward 4 flop + 1 exp per bin, backward 6 flop + 1 exp per bin, 6 flop per axis cosine.
WL, WA = 9, 33
F_FWD = 56 + 4 * WL + 12 * WA          # 488 flop per term
F_BWD = 61 + 6 * WL + 18 * WA          # 709 flop per term
F_FWD_DIST = 23 + 3 + 3 + 4 * WL       # distance encoding alone (no cosines, one window): 65 flop per term
X_TERM = 1 + WL + 3 * WA               # 109 exp per term, forward and backward alike
EPI_FWD = 4 * 2 * 16 * 64              # projection epilogue per (pair, head), four encodings
EPI_FWD_DIST = 2 * 16 * 64             # one encoding
PEAK_FP32_TFLOPS = 157.3               # published MI355X FP32 vector peak (packed FMA)
PEAK_FP32_UNPACKED = 78.6              # 256 CU x 64 lanes x 2 flop x 2.4 GHz, packed FP32 not used
PEAK_TRANS_TOPS = 9.8                  # quarter-rate transcendental unit
# HBM bytes per launch on the headline workload (batch 256, 64 + 64 bins, fused attention core), from rocprofv3 --pmc
# FETCH_SIZE / WRITE_SIZE (KiB per dispatch) scaled by what the same counters read for the 256 MiB device copy of
# --calibrate-copy; the figures and the commands are in TRAFFIC_SOURCE.  Other batch sizes or settings: null.
TRAFFIC_SOURCE = "profiles/fused_core_hbm_traffic_C3.md"
# forward 9 303.6 KiB x 2.0 + 92 229.7 KiB; backward 54 969.4 x 2.0 + 9 393.4; frame search 8 191.6 x 2.0 + 2 392.5
TRAFFIC_BYTES_PER_LAUNCH = {"fused_core_forward": 113.9e6, "fused_core_backward": 122.5e6, "frame_axes": 19.4e6}


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--batch", type=int, default=256)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-other-configs", action="store_true", help="skip the timed runs of C2, C4 and C5")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run one 256 MiB device-to-device copy (reference point for HBM traffic counters)")
    ap.add_argument("--torch-adamw", action="store_true", help="torch.optim.AdamW instead of the library's batched update")
    ap.add_argument("--no-fused-adamw", action="store_true", help="with --torch-adamw: the multi-tensor loop instead of the fused kernel")
    ap.add_argument("--no-graph", action="store_true",
                    help="launch every kernel from Python instead of replaying the step as one HIP graph")
    ap.add_argument("--two-step-core", action="store_true",
                    help="the reference's sequence of operators (lattice sums, then softmax attention) instead of "
                         "the fused attention core")
    ap.add_argument("--no-stats", action="store_true",
                    help="skip the passes that count lattice terms (their counters add atomics to the kernels, which a "
                         "profile of the kernels should not see); the roofline object is then null")
    ap.add_argument("--cpu-crystals", type=int, default=32, help="crystals of the batch in the CPU sample")
    ap.add_argument("--cpu-repeats", type=int, default=5, help="timed repetitions of the CPU sample (median)")
    return ap.parse_args()


def cpu_baseline(model, cb, mp, ncrys: int, repeats: int):
    """Forward + backward of the same model on the first ``ncrys`` crystals with the CPU oracle in the
    pure-PyTorch formulation of the reference (untruncated Gaussian bases)."""
    from oracle import cpu_model
    from crystalframer_amd.synthetic import CrystalBatch
    nat = int(cb.sizes[:ncrys].sum())
    sample = CrystalBatch(cb.x[:nat].cpu(), cb.pos[:nat].cpu(), cb.batch[:nat].cpu(),
                          cb.trans_vec[:ncrys].cpu(), cb.sizes[:ncrys].cpu())
    sd = {k: v.detach().cpu().clone() for k, v in model.state_dict().items()}
    cores = os.cpu_count() or 1
    torch.set_num_threads(cores)
    target = torch.zeros(ncrys, 1)
    times = []
    for rep in range(repeats + 1):
        leaves = {k: v.clone().requires_grad_(v.dtype.is_floating_point and "scale" not in k) for k, v in sd.items()}
        t0 = time.perf_counter()
        out = cpu_model.model_forward(leaves, sample, mp, dtype=torch.float32, windows="full")
        loss = torch.nn.functional.mse_loss(out, target)
        loss.backward()
        times.append(time.perf_counter() - t0)
    t = sorted(times[1:])[len(times[1:]) // 2]
    pairs = int((sample.sizes ** 2).sum())
    pairs_per_crystal_batch = float((cb.sizes.double() ** 2).mean())
    return {"value": ncrys / t, "unit": "crystals/s", "cores": cores, "kind": "port",
            "sample": f"first {ncrys} crystals of the batch ({nat} atoms, {pairs} atom pairs = {pairs / ncrys:.0f} per "
                      f"crystal; the whole batch has {pairs_per_crystal_batch:.0f} per crystal), 4-layer fwd+bwd, fp32 "
                      f"PyTorch restatement of the pure-PyTorch formulation (full Gaussian bases), median of "
                      f"{repeats} after 1 warm-up",
            "seconds_per_step": t}


def graphed(fn, warmup: int):
    """Capture ``fn`` (after ``warmup`` eager runs on the capture stream) and return the replay callable."""
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(max(warmup, 3)):
            fn()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):      # the stream of the warm-up: its library workspace is reused
        fn()
    for _ in range(2):
        graph.replay()
    torch.cuda.synchronize()
    return graph.replay


def timed(run, steps: int) -> float:
    """Seconds per call of ``run`` over exactly ``steps`` calls, device idle before and after."""
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        run()
    torch.cuda.synchronize()
    return (time.perf_counter() - t0) / steps


KERNELS = ("frame_axes", "framed_pe_forward", "framed_pe_backward", "fused_core_forward", "fused_core_backward")


def instrumented(fn, nprof: int, dev, count_terms: bool = True):
    """Run ``fn`` eagerly ``nprof`` times with the library's own HIP events around its lattice kernels and around
    every library call, then ``nprof`` times with the term counters.  Kept out of every timed region."""
    import crystalframer_amd as cf
    from crystalframer_amd import _lib
    KM = cf.KernelManager
    for what in KERNELS:                    # drop what earlier runs recorded
        _lib.read_kernel_timing(what)
    KM.EVENT_LOG = []
    _lib.kernel_timing(True)
    for _ in range(nprof):
        fn()
    torch.cuda.synchronize()
    _lib.kernel_timing(False)
    log, KM.EVENT_LOG = KM.EVENT_LOG, None
    kern_ms, kern_launches = {}, {}
    for what in KERNELS:
        total, count = _lib.read_kernel_timing(what)
        if count:
            kern_ms[what] = total / count
            kern_launches[what] = count // nprof
    stats = None
    if count_terms:
        KM.COLLECT_STATS = True
        _lib.read_stats(dev, reset=True)
        for _ in range(nprof):
            fn()
        torch.cuda.synchronize()
        KM.COLLECT_STATS = False
        stats = {k: v / nprof for k, v in _lib.read_stats(dev, reset=True).items() if not isinstance(v, list)}
    calls = {}
    for name, s, e in log:
        calls.setdefault(name, []).append(s.elapsed_time(e))
    return kern_ms, kern_launches, stats, calls


def lattice_roofline(kern_ms, kern_launches, stats, angle: bool):
    """Algorithmic flop of the reference formulation for the terms actually evaluated, per launch of the forward and
    of the backward lattice-sum kernel, over the kernel's own duration."""
    fwd = "fused_core_forward" if "fused_core_forward" in kern_ms else "framed_pe_forward"
    bwd = "fused_core_backward" if "fused_core_backward" in kern_ms else "framed_pe_backward"
    f_fwd, epi = (F_FWD, EPI_FWD) if angle else (F_FWD_DIST, EPI_FWD_DIST)
    out = {}
    if fwd in kern_ms:
        n = max(1, kern_launches[fwd])
        t = kern_ms[fwd] * 1e-3
        flop = stats["fwd_evaluated"] / n * f_fwd + stats["fwd_pairs"] / n * epi
        out["forward"] = {"kernel": fwd + "_kernel", "avg_launch_ms": kern_ms[fwd], "achieved": flop / t / 1e12,
                          "frac": flop / t / 1e12 / PEAK_FP32_TFLOPS, "terms_evaluated_per_launch": stats["fwd_evaluated"] / n,
                          "terms_in_box_per_launch": stats["fwd_in_box"] / n, "flop_per_launch": flop}
    if bwd in kern_ms and angle:
        n = max(1, kern_launches[bwd])
        t = kern_ms[bwd] * 1e-3
        flop = stats["bwd_evaluated"] / n * F_BWD + stats["bwd_pairs"] / n * 2 * EPI_FWD
        out["backward"] = {"kernel": bwd + "_kernel", "avg_launch_ms": kern_ms[bwd], "achieved": flop / t / 1e12,
                           "frac": flop / t / 1e12 / PEAK_FP32_TFLOPS, "terms_evaluated_per_launch": stats["bwd_evaluated"] / n,
                           "terms_in_box_per_launch": stats["bwd_in_box"] / n, "flop_per_launch": flop}
    return out


def other_config(name: str, dev, *, layers: int, backward: bool, angle_bins: int, steps: int):
    """One of the large configurations beside the headline one: the step as one HIP graph, timed by the host clock
    around ``steps`` replays; then the lattice kernels' own durations and term counts from instrumented eager runs."""
    from crystalframer_amd import latticeformer, params, synthetic
    torch.manual_seed(11)
    mp = params.ModelParams(num_layers=layers, value_pe_angle_real=angle_bins)
    model = latticeformer.Latticeformer(mp).to(dev)
    cb_cpu = synthetic.make_config(name, seed=123)
    cb = cb_cpu.to(dev)
    model.train()
    with torch.no_grad():
        model(cb)               # the first training-mode pass measures and stores the normalisation of alpha
    model.train(backward)
    B = cb_cpu.num_crystals
    target = torch.randn(B, 1, generator=torch.Generator().manual_seed(7)).to(dev)
    sink = torch.zeros((), device=dev)

    if backward:
        def fn():
            model.zero_grad(set_to_none=True)
            loss = torch.nn.functional.mse_loss(model(cb), target)
            loss.backward()
            sink.copy_(loss.detach())
    else:
        def fn():
            with torch.no_grad():
                sink.copy_(model(cb).sum())
    run = graphed(fn, 2)
    sec = timed(run, steps)
    kern_ms, kern_launches, stats, _ = instrumented(fn, 2, dev)
    roof = lattice_roofline(kern_ms, kern_launches, stats, angle_bins > 0)
    slow = max(roof.values(), key=lambda r: r["avg_launch_ms"]) if roof else None
    return {"workload": f"{name}: {B} crystals, {int(cb_cpu.pos.shape[0])} atoms, {int((cb_cpu.sizes ** 2).sum())} atom pairs; "
                        f"{layers}-layer max-frame model ({'64 + %d bins' % angle_bins if angle_bins else '64 distance bins, no angle encoding'}), "
                        f"{'forward + backward' if backward else 'forward only'}, one HIP graph per pass",
            "ms": sec * 1e3, "crystals_per_s": B / sec, "steps": steps,
            "lattice_kernel_ms": kern_ms,
            "lattice_kernel_frac": {k: r["frac"] for k, r in roof.items()},
            "slowest_lattice_kernel": None if slow is None else {"kernel": slow["kernel"], "frac": slow["frac"],
                                                                 "achieved_tflops": slow["achieved"]}}


def main():
    args = parse()
    if args.gpus != 1:
        print("bench.py measures one GPU: this build has no multi-GPU path (crystals would be sharded "
              "data-parallel, whole crystals per GPU, gradients all-reduced); run with --gpus 1", file=sys.stderr)
        sys.exit(2)
    if not torch.cuda.is_available():
        print("bench.py needs a HIP device", file=sys.stderr)
        sys.exit(2)
    import crystalframer_amd as cf
    from crystalframer_amd import attention, latticeformer, optim, params, synthetic
    KM = cf.KernelManager
    if args.two_step_core:
        attention.FUSED_CORE = False

    dev = torch.device("cuda:0")
    torch.manual_seed(123)
    mp = params.ModelParams()
    model = latticeformer.Latticeformer(mp).to(dev)
    model.train()
    cb_cpu = synthetic.make_config("C3", seed=123, num_crystals=args.batch)
    cb = cb_cpu.to(dev)
    target = torch.randn(args.batch, 1, generator=torch.Generator().manual_seed(7)).to(dev)
    use_graph = not args.no_graph
    # the library's AdamW: one launch for all parameter tensors (same update rule as torch.optim.AdamW, whose fused
    # multi-tensor kernel needs two launches of 43 us for the 65 small tensors of this model)
    if args.torch_adamw:
        opt = torch.optim.AdamW(model.parameters(), lr=5e-4, betas=(0.9, 0.98), weight_decay=1e-5,
                                capturable=use_graph, fused=not args.no_fused_adamw)
    else:
        opt = optim.AdamW(model.parameters(), lr=5e-4, betas=(0.9, 0.98), weight_decay=1e-5)
    # the tie-breaking noise of the frame search: seed word on the device, advanced by every call, so
    # that replays of the captured step draw fresh noise like separate launches do
    KM.NOISE_SEED = 20240607
    KM.NOISE_SEED_DEVICE = torch.zeros(1, dtype=torch.int64, device=dev)
    loss_out = torch.zeros((), device=dev)

    def step():
        opt.zero_grad(set_to_none=True)
        out = model(cb)
        loss = torch.nn.functional.mse_loss(out, target)
        loss.backward()
        opt.step()
        loss_out.copy_(loss.detach())

    if use_graph:
        # the whole training step (geometry, 4 layers forward, loss, backward, AdamW) as ONE HIP graph:
        # Python cannot issue the step's launches as fast as the GPU retires them
        run_step = graphed(step, args.warmup)
    else:
        run_step = step
        for _ in range(args.warmup):
            step()
    torch.cuda.synchronize()

    # ---- timed region: exactly K steps
    t0 = time.perf_counter()
    for _ in range(args.steps):
        run_step()
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    final_loss = float(loss_out)
    ms_per_step = dt / args.steps * 1e3
    crystals_per_s = args.batch / (dt / args.steps)

    # ---- instrumented passes over the same step, outside the timed region
    nprof = min(args.steps, 5)
    kern_ms, kern_launches, stats, calls = instrumented(step, nprof, dev, count_terms=not args.no_stats)
    avg_ms = {k: sum(v) / len(v) for k, v in calls.items()}
    launches = {k: len(v) // nprof for k, v in calls.items()}
    lib_ms_per_step = sum(sum(v) for v in calls.values()) / nprof
    if args.calibrate_copy:
        src = torch.empty(64 * 1024 * 1024, dtype=torch.float32, device=dev).normal_()
        dst = torch.empty_like(src)
        dst.copy_(src)
        torch.cuda.synchronize()
    if stats is None:
        print(json.dumps({"metric": f"crystals/s fwd+bwd, 4-layer max-frame, batch {args.batch}", "value": crystals_per_s,
                          "unit": "crystals/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
                          "ms_per_step": ms_per_step, "higher_is_better": True, "roofline": None,
                          "lattice_kernel_ms": kern_ms, "library_call_ms": avg_ms}))
        return
    roof = lattice_roofline(kern_ms, kern_launches, stats, True)
    dom = max(roof.values(), key=lambda r: r["avg_launch_ms"])
    fused = "fused_core_forward" in kern_ms
    traffic = TRAFFIC_BYTES_PER_LAUNCH.get(dom["kernel"][:-len("_kernel")]) if (args.batch == 256 and fused) else None
    roofline = {
        "kernel": dom["kernel"], "bound": "valu-issue",
        "achieved": dom["achieved"], "peak": PEAK_FP32_TFLOPS, "unit": "TFLOP/s", "frac": dom["frac"], "traffic": traffic,
        "traffic_source": TRAFFIC_SOURCE if traffic is not None else None,
        "bound_detail": "ALGORITHMIC FP32 flop of the reference formulation (what its kernels would execute for the terms "
                        "this kernel evaluates) against the published 157.3 TFLOP/s vector peak.  The kernel does not "
                        "execute that many: the angle encoding is scattered as 5 local moments per axis instead of a "
                        "33-bin window and the projection runs once per (atom, head) in a separate MFMA kernel.  What "
                        "binds it is the issue of vector instructions, few of which are multiply-adds (one wavefront per "
                        "(atom, head), 12.5 pairs on average): vector ALUs issuing 76 % of the kernel's time with 79 % "
                        "of the lanes active, HBM at a quarter of its peak (profiles/fused_core_valu_lds_counters_C3.md)",
        "both_kernels": {k: {"kernel": r["kernel"], "achieved": r["achieved"], "frac": r["frac"],
                             "avg_launch_ms": r["avg_launch_ms"]} for k, r in roof.items()},
        "frac_of_unpacked_fp32_peak": dom["achieved"] / PEAK_FP32_UNPACKED,
        "transcendental_frac": dom["terms_evaluated_per_launch"] * X_TERM / (dom["avg_launch_ms"] * 1e-3) / 1e12 / PEAK_TRANS_TOPS,
        "avg_launch_ms": dom["avg_launch_ms"],
        "terms_evaluated_per_launch": dom["terms_evaluated_per_launch"],
        "note": "algorithmic flop of the reference formulation (709 bwd / 488 fwd per term, 109 exp) x terms "
                "actually evaluated after pruning, + one projection epilogue per (pair, head) and encoding (two for the "
                "backward); duration from HIP events recorded by the library around this kernel alone, on the stream it "
                "is launched on",
    }
    terms = {}
    for k, r in roof.items():
        t = r["avg_launch_ms"] * 1e-3
        terms[k + "_terms_in_box_per_s"] = r["terms_in_box_per_launch"] / t
        terms[k + "_terms_evaluated_per_s"] = r["terms_evaluated_per_launch"] / t
    if "forward" in roof:
        terms["evaluated_fraction"] = roof["forward"]["terms_evaluated_per_launch"] / max(1.0, roof["forward"]["terms_in_box_per_launch"])

    result = {
        "metric": f"crystals/s fwd+bwd, 4-layer max-frame, batch {args.batch}",
        "value": crystals_per_s, "unit": "crystals/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": ms_per_step, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32", "data": "synthetic",
        "config": {"workload": "C3: 4-layer CrystalFramer max-frame encoder + mean pooling + MLP head, one training "
                               "step (forward, MSE, backward, AdamW), fp32",
                   "global_batch": args.batch, "atoms": int(cb.pos.shape[0]),
                   "atom_pairs": int((cb_cpu.sizes ** 2).sum()), "heads": 8, "head_dim": 16,
                   "dist_bins": 64, "angle_bins": 64, "adaptive_cutoff_sigma": -3.5, "prune_log2": KM.PRUNE_LOG2,
                   "attention_core": "fused (one histogram per (atom, head))" if fused else "two-step (reference's operators)",
                   "windows": "distance 9 bins, angle basis untruncated" if fused else "reference (9/33 bins)",
                   "optimizer": "adamw", "parallelism": "single GPU",
                   "launch": "one HIP graph per step" if use_graph else "eager"},
        "final_loss": final_loss,
        "roofline": roofline,
        "lattice_terms": terms,
        "lattice_kernel_ms": kern_ms, "library_call_ms": avg_ms, "library_calls_per_step": launches,
        "library_ms_per_step": lib_ms_per_step,
    }
    if args.calibrate_copy:
        result["calibrate_copy_bytes"] = int(src.numel() * 4)
    if not args.no_other_configs:
        # the other large configurations, each timed by this process's clock around graph replays
        del opt
        other = {}
        other["C2"] = other_config("C2", dev, layers=1, backward=True, angle_bins=64, steps=20)
        other["C4"] = other_config("C4", dev, layers=1, backward=True, angle_bins=64, steps=10)
        other["C5"] = other_config("C5", dev, layers=4, backward=False, angle_bins=64, steps=10)
        other["C5_no_angle"] = other_config("C5", dev, layers=4, backward=False, angle_bins=0, steps=10)
        result["other_configs"] = other
    if not args.no_cpu_baseline:
        result["cpu_baseline"] = cpu_baseline(model, cb_cpu, mp, min(args.cpu_crystals, args.batch), args.cpu_repeats)
    print(json.dumps(result))


if __name__ == "__main__":
    main()
