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
F_FRAME = 25 + 24 + 38                 # the three sweeps of the frame search: 87 flop per term looked at
F_FWD_DIST = 23 + 3 + 3 + 4 * WL       # distance encoding alone (no cosines, one window): 65 flop per term
F_BWD_DIST = 23 + 3 + 3 + 8 + 6 * WL   # ... backward: 91 flop per term
X_TERM = 1 + WL + 3 * WA               # 109 exp per term, forward and backward alike
EPI_FWD = 4 * 2 * 16 * 64              # projection epilogue per (pair, head), four encodings
EPI_FWD_DIST = 2 * 16 * 64             # one encoding
PEAK_FP32_TFLOPS = 157.3               # published MI355X FP32 vector peak (packed FMA)
PEAK_FP32_UNPACKED = 78.6              # 256 CU x 64 lanes x 2 flop x 2.4 GHz, packed FP32 not used
PEAK_TRANS_TOPS = 9.8                  # quarter-rate transcendental unit
# What rocprofv3 counted on the headline workload (batch 256, 64 + 64 bins, fused attention core): HBM bytes per
# launch of every kernel of the path (--pmc FETCH_SIZE / WRITE_SIZE scaled by what the same counters read for the
# 256 MiB device copy of --calibrate-copy) and the vector-ALU counters of the lattice kernels.  The summaries hold
# the commands, the raw readings and, at their end, the `key = value` lines read here.  Other batch sizes or
# settings: null.
TRAFFIC_SOURCE = "profiles/fused_core_hbm_traffic_C3.md"
COUNTER_SOURCE = "profiles/fused_core_valu_lds_counters_C3.md"

# The kernels that execute the work counted for a path, by the names the library times them under
# (cfh_timing_enable): the algorithmic flop of a path are divided by the SUM of their durations.
PATHS = {
    "forward": {
        "fused": ("core_tables", "core_prepare", "frame_axes", "fused_core_forward", "core_project"),
        "two_step": ("frame_axes", "framed_pe_forward"),
    },
    "backward": {
        "fused": ("core_prepare_bwd", "core_gbuild", "fused_core_backward", "core_bwd_col", "core_weight_gradients"),
        "two_step": ("framed_pe_backward",),
    },
}
KERNEL_NAMES = {
    "core_tables": "sorted_shifts_kernel + pair_nearest_kernel (once per batch)",
    "core_prepare": "core_prepare_wcat_kernel", "frame_axes": "frame_axes_kernel",
    "fused_core_forward": "fused_core_fwd_kernel", "core_project": "core_project_kernel",
    "core_prepare_bwd": "core_wcat_kernel / prepare_items_kernel (only when the forward's are not kept)",
    "core_gbuild": "core_gbuild_kernel", "fused_core_backward": "fused_core_bwd_kernel",
    "core_bwd_col": "dpa_bwd_col_kernel",
    "core_weight_gradients": "core_gwcat_multi_kernel + core_gw_finish_multi_kernel (once per step, all layers)",
    "framed_pe_forward": "framed_pe_fwd_kernel", "framed_pe_backward": "framed_pe_bwd_saved_kernel + gw_from_histograms_kernel",
}


def read_profile_table(path: str) -> dict:
    """The `key = value` lines of a committed profile summary (numbers only)."""
    import re
    out = {}
    full = os.path.join(ROOT, path)
    if not os.path.exists(full):
        return out
    for line in open(full):
        m = re.match(r"^\s*([A-Za-z_][A-Za-z0-9_.]*)\s*=\s*([-+0-9.eE]+)\s*$", line)
        if m:
            out[m.group(1)] = float(m.group(2))
    return out


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
    ap.add_argument("--core-distance-window", type=int, choices=(9, 11), default=None,
                    help="distance window of the fused core: 11 bins (+-5 sigma, the default: full-basis semantics) or the "
                         "9 bins of the reference's CUDA kernels")
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


KERNELS = tuple(KERNEL_NAMES)


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
            kern_launches[what] = count / nprof
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


def lattice_roofline(kern_ms, kern_launches, stats, angle: bool, items_per_launch: int, angle_bins: int = 64):
    """Per pass (all layers of one step), forward and backward: algorithmic flop over the SUM of the durations of
    every kernel that executes part of that work, each measured by the library with HIP events on its launch stream.
    Algorithmic flop = the per-term counts above x the terms actually evaluated, 87 flop per candidate the frame
    search looks at, and the projections as this build's formulation makes them (one per (atom, head) =
    ``items_per_launch`` per layer for the fused core; one per (pair, head) and encoding for the two-step operators).
    The projections of the reference's formulation (per pair) are reported beside it, not counted: the fused core does
    not execute them."""
    fused = "fused_core_forward" in kern_ms
    kind = "fused" if fused else "two_step"
    f_fwd, f_bwd, epi = (F_FWD, F_BWD, EPI_FWD) if angle else (F_FWD_DIST, F_BWD_DIST, EPI_FWD_DIST)
    if angle and angle_bins == 16:      # the whole 16-bin basis per axis instead of a 33-bin window
        f_fwd, f_bwd, epi = 56 + 4 * WL + 12 * 16, 61 + 6 * WL + 18 * 16, 2 * 16 * (64 + 3 * 16)
    if not angle:
        angle_bins = 0
    out = {}
    for path, (ev, pairs) in (("forward", ("fwd_evaluated", "fwd_pairs")), ("backward", ("bwd_evaluated", "bwd_pairs"))):
        names = [k for k in PATHS[path][kind] if k in kern_ms]
        main = ("fused_core_" if fused else "framed_pe_") + path
        if main not in kern_ms:
            continue
        per_kernel = {k: {"kernel": KERNEL_NAMES[k], "avg_launch_ms": kern_ms[k], "launches_per_step": kern_launches[k],
                          "ms_per_step": kern_ms[k] * kern_launches[k]} for k in names}
        t = sum(v["ms_per_step"] for v in per_kernel.values()) * 1e-3
        per_term = f_fwd if path == "forward" else f_bwd
        passes = 1 if path == "forward" else 2          # backward: gradient of the histogram and weight gradients
        flop_terms = stats[ev] * per_term
        frame_terms = (stats.get("frame1_scanned", 0.0) + stats.get("frame2_scanned", 0.0)) if (path == "forward" and angle) else 0.0
        flop_frames = frame_terms * F_FRAME
        n = max(1.0, kern_launches[main])
        # projections: the reference's formulation makes one per (pair, head) and encoding; the fused core makes one
        # per (atom, head) over its histogram of hw words (64 distance bins + 3 axes x 5 moments x 64 bins)
        flop_epi_reference = stats[pairs] * epi * passes
        if fused:
            hw = {64: 1024, 16: 128}.get(angle_bins, 64)
            flop_epi = items_per_launch * n * 2 * 16 * hw * passes
        else:
            flop_epi = flop_epi_reference
        flop = flop_terms + flop_frames + flop_epi
        out[path] = {"kernels": per_kernel, "ms_per_step": t * 1e3, "flop_per_step": flop,
                     "flop_breakdown": {"lattice_terms": flop_terms, "frame_search": flop_frames, "projections": flop_epi,
                                        "projections_of_the_reference_formulation": flop_epi_reference},
                     "achieved": flop / t / 1e12, "frac": flop / t / 1e12 / PEAK_FP32_TFLOPS,
                     "reference_equivalent_tflops": (flop_terms + flop_frames + flop_epi_reference) / t / 1e12,
                     "main_kernel": KERNEL_NAMES[main], "main_kernel_avg_launch_ms": kern_ms[main],
                     "terms_evaluated_per_launch": stats[ev] / n,
                     "terms_in_box_per_launch": stats["fwd_in_box" if path == "forward" else "bwd_in_box"] / n,
                     "frame_candidates_per_launch": frame_terms / n,
                     "exp_per_step": stats[ev] * (X_TERM if angle else 1 + WL)}
    return out


def other_config(name: str, dev, *, layers: int, backward: bool, angle_bins: int, steps: int, **model_kw):
    """One of the large configurations beside the headline one: the step as one HIP graph, timed by the host clock
    around ``steps`` replays; then the lattice kernels' own durations and term counts from instrumented eager runs."""
    from crystalframer_amd import latticeformer, params, synthetic
    torch.manual_seed(11)
    mp = params.ModelParams(num_layers=layers, value_pe_angle_real=angle_bins, **model_kw)
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
    roof = lattice_roofline(kern_ms, kern_launches, stats, angle_bins > 0, int(cb_cpu.pos.shape[0]) * mp.head_num, angle_bins)
    return {"workload": f"{name}: {B} crystals, {int(cb_cpu.pos.shape[0])} atoms, {int((cb_cpu.sizes ** 2).sum())} atom pairs; "
                        f"{layers}-layer max-frame model ({'64 + %d bins' % angle_bins if angle_bins else '64 distance bins, no angle encoding'}), "
                        f"{'forward + backward' if backward else 'forward only'}, one HIP graph per pass",
            "ms": sec * 1e3, "crystals_per_s": B / sec, "steps": steps,
            "lattice_kernel_ms": kern_ms,
            "paths": {k: {"frac": r["frac"], "achieved_tflops": r["achieved"], "ms_per_step": r["ms_per_step"],
                          "flop_breakdown": r["flop_breakdown"], "reference_equivalent_tflops": r["reference_equivalent_tflops"],
                          "terms_evaluated_per_launch": r["terms_evaluated_per_launch"],
                          "main_kernel_avg_launch_ms": r["main_kernel_avg_launch_ms"]} for k, r in roof.items()}}


def build_step(args, dev, mp, cb, target):
    """Model, optimizer and the training step of the headline workload."""
    import crystalframer_amd as cf
    from crystalframer_amd import latticeformer, optim
    KM = cf.KernelManager
    torch.manual_seed(123)
    model = latticeformer.Latticeformer(mp).to(dev)
    model.train()
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

    return model, step, loss_out


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
    from crystalframer_amd import _lib, attention, params, synthetic
    KM = cf.KernelManager
    if args.two_step_core:
        attention.FUSED_CORE = False
    if args.core_distance_window is not None:
        KM.CORE_WINDOW_MODE = _lib.CFH_WINDOW_WIDE if args.core_distance_window == 11 else _lib.CFH_WINDOW_REFERENCE

    dev = torch.device("cuda:0")
    mp = params.ModelParams()
    cb_cpu = synthetic.make_config("C3", seed=123, num_crystals=args.batch)
    cb = cb_cpu.to(dev)
    target = torch.randn(args.batch, 1, generator=torch.Generator().manual_seed(7)).to(dev)
    use_graph = not args.no_graph
    model, step, loss_out = build_step(args, dev, mp, cb, target)

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
    roof = lattice_roofline(kern_ms, kern_launches, stats, True, int(cb.pos.shape[0]) * mp.head_num)
    dom_name, dom = max(roof.items(), key=lambda kv: kv[1]["ms_per_step"])
    fused = "fused_core_forward" in kern_ms
    wide = KM.CORE_WINDOW_MODE == _lib.CFH_WINDOW_WIDE
    headline_setting = args.batch == 256 and fused and wide
    # counters of the committed profiles (headline workload and setting only)
    tr = read_profile_table(TRAFFIC_SOURCE) if headline_setting else {}
    ct = read_profile_table(COUNTER_SOURCE) if headline_setting else {}

    def path_traffic(r):
        """HBM bytes per step of a path's kernels: bytes per launch (profile) x launches per step (this run)."""
        total = 0.0
        for k, v in r["kernels"].items():
            key = "hbm_bytes_per_launch." + k
            if key not in tr:
                return None
            total += tr[key] * v["launches_per_step"]
        return total

    def executed(path):
        """What the main kernel of a path executed, by the counter profile: fraction of its time the vector ALUs
        issue, lanes active, transcendental rate against the quarter-rate unit."""
        pre = "counters." + ("fused_core_forward" if path == "forward" else "fused_core_backward") + "."
        keys = ("valu_issue_frac", "valu_issue_frac_of_busy_cycles", "valu_lanes_active_frac", "valu_wave_insts_per_launch", "trans_wave_insts_per_launch",
                "salu_wave_insts_per_launch", "mfma_wave_insts_per_launch", "avg_launch_us")
        got = {k: ct[pre + k] for k in keys if pre + k in ct}
        if "trans_wave_insts_per_launch" in got and "avg_launch_us" in got:
            got["transcendental_frac_of_9p8_T_per_s"] = (got["trans_wave_insts_per_launch"] * 64 / (got["avg_launch_us"] * 1e-6)
                                                          / 1e12 / PEAK_TRANS_TOPS)
        return got or None

    traffic = path_traffic(dom)
    roofline = {
        "kernel": dom_name + " pass of the lattice path: " + " + ".join(v["kernel"] for v in dom["kernels"].values()),
        "bound": "valu",
        "achieved": dom["achieved"], "peak": PEAK_FP32_TFLOPS, "unit": "TFLOP/s", "frac": dom["frac"],
        "traffic": traffic, "traffic_unit": "HBM bytes per step over the kernels named (4 launches each but for the "
                                            "once-per-step ones)" if traffic is not None else None,
        "traffic_source": TRAFFIC_SOURCE if traffic is not None else None,
        "executed": executed(dom_name), "executed_source": COUNTER_SOURCE if ct else None,
        "bound_detail": "achieved = algorithmic FP32 flop divided by the SUM of the durations of all kernels that execute "
                        "them, against the published 157.3 TFLOP/s (packed FP32, which this build does not use: 78.6 "
                        "unpacked).  Algorithmic = 488 (forward) / 709 (backward) flop per lattice term evaluated (the "
                        "reference's windowed formulation), 87 per candidate of the frame search, and the projections as "
                        "made here, once per (atom, head) over 1024 histogram words (the reference's one-per-pair "
                        "projections are NOT counted; with them: reference_equivalent_tflops).  The lattice kernels "
                        "execute fewer flop per term than that (5 local moments per axis instead of a 33-bin window); "
                        "what they executed is under `executed`, from rocprofv3 counters of the same workload",
        "paths": {k: {"frac": r["frac"], "achieved": r["achieved"], "ms_per_step": r["ms_per_step"],
                      "flop_per_step": r["flop_per_step"], "flop_breakdown": r["flop_breakdown"],
                      "reference_equivalent_tflops": r["reference_equivalent_tflops"],
                      "frac_of_unpacked_fp32_peak": r["achieved"] / PEAK_FP32_UNPACKED,
                      "algorithmic_exp_frac_of_9p8_T_per_s": r["exp_per_step"] / (r["ms_per_step"] * 1e-3) / 1e12 / PEAK_TRANS_TOPS,
                      "hbm_bytes_per_step": path_traffic(r),
                      "hbm_GB_per_s": (path_traffic(r) / (r["ms_per_step"] * 1e-3) / 1e9) if path_traffic(r) else None,
                      "executed": executed(k),
                      "kernels": r["kernels"]} for k, r in roof.items()},
        "avg_launch_ms": dom["main_kernel_avg_launch_ms"],
        "terms_evaluated_per_launch": dom["terms_evaluated_per_launch"],
        "note": "durations from HIP events that the library records around each of its kernels on the stream it "
                "launches them on, in eager re-runs of the same steps outside the timed region; terms counted by the "
                "kernels in separate instrumented passes",
    }
    terms = {}
    for k, r in roof.items():
        t = r["main_kernel_avg_launch_ms"] * 1e-3
        terms[k + "_terms_in_box_per_s"] = r["terms_in_box_per_launch"] / t
        terms[k + "_terms_evaluated_per_s"] = r["terms_evaluated_per_launch"] / t
        terms[k + "_terms_evaluated_per_s_over_the_path"] = (r["terms_evaluated_per_launch"] *
                                                            r["kernels"][[n for n in r["kernels"] if n.endswith(k)][0]]["launches_per_step"]
                                                            / (r["ms_per_step"] * 1e-3))
    if "forward" in roof:
        terms["evaluated_fraction"] = roof["forward"]["terms_evaluated_per_launch"] / max(1.0, roof["forward"]["terms_in_box_per_launch"])

    if fused:
        windows = ("distance 11 bins (+-5 sigma: a dropped bin is below 4e-6 of a basis function's peak), angle basis "
                   "untruncated: the full Gaussian bases of the reference's pure-PyTorch formulation") if wide else \
                  "distance 9 bins (the +-4 sigma window of the reference's CUDA kernels), angle basis untruncated"
    else:
        windows = "reference (9/33 bins)"
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
                   "windows": windows,
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
        del step, run_step
        other = {}
        if fused and wide and use_graph:
            # the same step with the 9-bin distance window of the reference's CUDA kernels: what the wider window costs
            KM.CORE_WINDOW_MODE = _lib.CFH_WINDOW_REFERENCE
            _, step9, _ = build_step(args, dev, mp, cb, target)
            sec9 = timed(graphed(step9, args.warmup), args.steps)
            KM.CORE_WINDOW_MODE = _lib.CFH_WINDOW_WIDE
            other["C3_distance_window_9_bins"] = {"workload": "the headline step with the +-4 sigma distance window (9 bins) "
                                                              "instead of the +-5 sigma one (11 bins)",
                                                  "ms": sec9 * 1e3, "crystals_per_s": args.batch / sec9, "steps": args.steps}
            del step9
        # the reference's lightweight setting (train_jarvis_time.sh:40-57): 16 angle bins, sigma one bin
        other["C3_lightweight"] = other_config("C3", dev, layers=4, backward=True, angle_bins=16, steps=20,
                                               value_pe_angle_wscale=1.0, value_pe_dist_coef=1.5, value_pe_angle_coef=6.0)
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
