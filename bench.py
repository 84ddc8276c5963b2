#!/usr/bin/env python3
"""Benchmark of the periodic-attention hot path on one MI355X.

One "step" is one training step (forward, MSE loss, backward, AdamW update) of the 4-layer
CrystalFramer max-frame model over one batch of 256 synthetic crystals that is already resident in
HBM (configuration C3: the 4-layer max-frame model at batch 256; fp32, random-init weights).  Prints ONE JSON line with
crystals/s, the roofline figures of the dominant kernel measured with HIP events inside the timed
steps, and the CPU baseline (the PyTorch restatement of the reference's pure-PyTorch formulation,
timed on the host cores on a bounded sample of the same batch).

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-cpu-baseline]
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
X_TERM = 1 + WL + 3 * WA               # 109 exp per term, forward and backward alike
F_FRAME = 87                           # three frame-search sweeps
EPI_FWD = 4 * 2 * 16 * 64              # projection epilogue per (pair, head)
PEAK_FP32_TFLOPS = 157.3               # published MI355X FP32 vector peak (packed FMA)
PEAK_FP32_UNPACKED = 78.6              # 256 CU x 64 lanes x 2 flop x 2.4 GHz, packed FP32 not used
PEAK_TRANS_TOPS = 9.8                  # quarter-rate transcendental unit
# HBM bytes per launch of the dominant kernel on this workload, from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE
# (KiB per dispatch) scaled by what the same counters read for the 256 MiB device copy of --calibrate-copy
# (FETCH_SIZE reads 128 MiB for it: factor 2.0; WRITE_SIZE reads 256 MiB: factor 1.0); see profiles/.
# With the forward keeping its window histograms for the backward (KernelManager.SAVE_HISTOGRAMS, the default):
# forward 3 398 KiB x 2.0 fetched + 261 810 KiB written (243.9 MB of that are the histograms, E x H x 4 x 64
# floats); backward: the gather-only kernel 25 477 KiB x 2.0 fetched and under 2 MB written, the weight-gradient
# kernel beside it on the second stream 133 999 KiB x 2.0 fetched (the histograms again) + 16 384 KiB written (its
# per-wavefront partials).
TRAFFIC_BYTES_PER_LAUNCH = {"framed_pe_backward": 52.2e6 + 291.2e6, "framed_pe_forward": 275.0e6}


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--batch", type=int, default=256)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run one 256 MiB device-to-device copy (reference point for HBM traffic counters)")
    ap.add_argument("--no-fused-adamw", action="store_true", help="PyTorch's multi-tensor AdamW instead of the fused kernel")
    ap.add_argument("--no-graph", action="store_true",
                    help="launch every kernel from Python instead of replaying the step as one HIP graph")
    ap.add_argument("--cpu-crystals", type=int, default=12, help="crystals of the batch in the CPU sample")
    return ap.parse_args()


def cpu_baseline(model, cb, mp, ncrys: int):
    """Forward + backward of the same model on the first ``ncrys`` crystals with the CPU oracle."""
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
    for rep in range(3):
        leaves = {k: v.clone().requires_grad_(v.dtype.is_floating_point and "scale" not in k) for k, v in sd.items()}
        t0 = time.perf_counter()
        out = cpu_model.model_forward(leaves, sample, mp, dtype=torch.float32)
        loss = torch.nn.functional.mse_loss(out, target)
        loss.backward()
        times.append(time.perf_counter() - t0)
    t = sorted(times[1:])[len(times[1:]) // 2] if len(times) > 1 else times[0]
    pairs = int((sample.sizes ** 2).sum())
    return {"value": ncrys / t, "unit": "crystals/s", "cores": cores, "kind": "port",
            "sample": f"first {ncrys} crystals of the batch ({nat} atoms, {pairs} atom pairs), 4-layer fwd+bwd, "
                      f"fp32 PyTorch restatement of the pure-PyTorch formulation, median of {len(times) - 1} after 1 warm-up",
            "seconds_per_step": t}


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
    from crystalframer_amd import _lib, latticeformer, params, synthetic
    KM = cf.KernelManager

    dev = torch.device("cuda:0")
    torch.manual_seed(123)
    mp = params.ModelParams()
    model = latticeformer.Latticeformer(mp).to(dev)
    model.train()
    cb_cpu = synthetic.make_config("C3", seed=123, num_crystals=args.batch)
    cb = cb_cpu.to(dev)
    target = torch.randn(args.batch, 1, generator=torch.Generator().manual_seed(7)).to(dev)
    use_graph = not args.no_graph
    # fused=True: PyTorch's single-kernel AdamW (same update rule as the default multi-tensor loop)
    opt = torch.optim.AdamW(model.parameters(), lr=5e-4, betas=(0.9, 0.98), weight_decay=1e-5,
                            capturable=use_graph, fused=not args.no_fused_adamw)
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
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            for _ in range(max(args.warmup, 3)):
                step()
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=side):      # the stream of the warm-up: its library workspace is reused
            step()
        run_step = graph.replay
        for _ in range(2):
            run_step()
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

    # ---- a second, instrumented pass over the same steps: HIP events around every library call on
    #      its stream, and term counters; kept out of the timed region so that it cannot perturb it
    KM.EVENT_LOG = []
    _lib.kernel_timing(True)          # the library's own event bracket around each lattice-sum kernel
    nprof = min(args.steps, 5)
    for _ in range(nprof):
        step()
    torch.cuda.synchronize()
    _lib.kernel_timing(False)
    log, KM.EVENT_LOG = KM.EVENT_LOG, None
    kern_ms = {}
    for what in ("frame_axes", "framed_pe_forward", "framed_pe_backward", "fused_core_forward", "fused_core_backward"):
        total, count = _lib.read_kernel_timing(what)
        if count:
            kern_ms[what] = total / count
    # ---- and a third one that counts translations (separately: the counters add a few atomics)
    KM.COLLECT_STATS = True
    _lib.read_stats(dev, reset=True)
    for _ in range(nprof):
        step()
    torch.cuda.synchronize()
    KM.COLLECT_STATS = False
    stats = _lib.read_stats(dev, reset=True)
    per_kernel = {}
    for name, s, e in log:
        per_kernel.setdefault(name, []).append(s.elapsed_time(e))
    avg_ms = {k: sum(v) / len(v) for k, v in per_kernel.items()}
    launches = {k: len(v) // nprof for k, v in per_kernel.items()}
    lib_ms_per_step = sum(sum(v) for v in per_kernel.values()) / nprof

    fused = "fused_core_forward" in kern_ms
    if fused:
        kern_ms["framed_pe_forward"] = kern_ms["fused_core_forward"]
        kern_ms["framed_pe_backward"] = kern_ms["fused_core_backward"]
    nlaunch_bwd = max(1, len(per_kernel.get("framed_pe_backward", [])) + len(per_kernel.get("fused_core_backward", [])))
    nlaunch_fwd = max(1, len(per_kernel.get("framed_pe_forward", [])) + len(per_kernel.get("frame_axes_framed_pe_forward", []))
                      + len(per_kernel.get("fused_core_forward", [])))
    bwd_eval = stats["bwd_evaluated"] / nlaunch_bwd          # terms evaluated per launch
    bwd_box = stats["bwd_in_box"] / nlaunch_bwd              # terms in the reference's boxes per launch
    bwd_pairs = stats["bwd_pairs"] / nlaunch_bwd
    fwd_eval = stats["fwd_evaluated"] / nlaunch_fwd
    fwd_box = stats["fwd_in_box"] / nlaunch_fwd
    fwd_pairs = stats["fwd_pairs"] / nlaunch_fwd
    t_bwd = kern_ms.get("framed_pe_backward", float("nan")) * 1e-3
    t_fwd = kern_ms.get("framed_pe_forward", float("nan")) * 1e-3
    flop_bwd = bwd_eval * F_BWD + bwd_pairs * 2 * EPI_FWD    # terms actually evaluated + epilogues
    flop_fwd = fwd_eval * F_FWD + fwd_pairs * EPI_FWD
    dominant = "framed_pe_backward" if t_bwd >= t_fwd else "framed_pe_forward"
    flop_dom, t_dom, eval_dom = (flop_bwd, t_bwd, bwd_eval) if dominant == "framed_pe_backward" else (flop_fwd, t_fwd, fwd_eval)
    achieved = flop_dom / t_dom / 1e12
    roofline = {
        "kernel": dominant + "_kernel", "bound": "mfma", "achieved": achieved, "peak": PEAK_FP32_TFLOPS,
        "unit": "TFLOP/s", "frac": achieved / PEAK_FP32_TFLOPS, "traffic": TRAFFIC_BYTES_PER_LAUNCH.get(dominant),
        "bound_detail": "FP32 arithmetic (vector + a little MFMA) against the published 157.3 TFLOP/s; HBM traffic "
                        "(the kept window histograms) runs at 15-18 % of the HBM peak; in practice the forward is "
                        "limited by LDS atomic throughput and bank conflicts, the backward (a gather-only kernel "
                        "with the weight-gradient kernel beside it on a second stream) by instruction issue",
        "both_kernels": {
            "framed_pe_forward": {"achieved": flop_fwd / t_fwd / 1e12, "frac": flop_fwd / t_fwd / 1e12 / PEAK_FP32_TFLOPS,
                                  "avg_launch_ms": t_fwd * 1e3},
            # the gather-only kernel's duration; the weight-gradient kernel (its share of the flop: one projection
            # epilogue per (pair, head)) runs inside that time on the second stream
            "framed_pe_backward": {"achieved": flop_bwd / t_bwd / 1e12, "frac": flop_bwd / t_bwd / 1e12 / PEAK_FP32_TFLOPS,
                                   "avg_launch_ms": t_bwd * 1e3},
        },
        "frac_of_unpacked_fp32_peak": achieved / PEAK_FP32_UNPACKED,
        "transcendental_frac": eval_dom * X_TERM / t_dom / 1e12 / PEAK_TRANS_TOPS,
        "avg_launch_ms": t_dom * 1e3,
        "terms_evaluated_per_launch": eval_dom,
        "note": "algorithmic flop of the reference formulation (709 bwd / 488 fwd per term, 109 exp) x terms "
                "actually evaluated after pruning, + projection epilogues; duration from HIP events recorded by "
                "the library around this kernel alone, on the stream it is launched on",
    }
    terms = {
        "forward_terms_in_box_per_s": fwd_box / t_fwd, "forward_terms_evaluated_per_s": fwd_eval / t_fwd,
        "backward_terms_in_box_per_s": bwd_box / t_bwd, "backward_terms_evaluated_per_s": bwd_eval / t_bwd,
        "evaluated_fraction": fwd_eval / max(1.0, fwd_box),
    }

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
                   "windows": "reference (9/33 bins)", "optimizer": "adamw", "parallelism": "single GPU",
                   "launch": "one HIP graph per step" if use_graph else "eager"},
        "final_loss": final_loss,
        "roofline": roofline,
        "lattice_terms": terms,
        "lattice_kernel_ms": kern_ms, "library_call_ms": avg_ms, "library_calls_per_step": launches,
        "library_ms_per_step": lib_ms_per_step,
    }
    if args.calibrate_copy:
        src = torch.empty(64 * 1024 * 1024, dtype=torch.float32, device=dev).normal_()
        dst = torch.empty_like(src)
        dst.copy_(src)
        torch.cuda.synchronize()
        result["calibrate_copy_bytes"] = int(src.numel() * 4)
    if not args.no_cpu_baseline:
        result["cpu_baseline"] = cpu_baseline(model, cb_cpu, mp, min(args.cpu_crystals, args.batch))
    print(json.dumps(result))


if __name__ == "__main__":
    main()
