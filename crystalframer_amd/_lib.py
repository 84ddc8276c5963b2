"""ctypes binding of libcrystalframer_hip.so (the C ABI declared in include/crystalframer_hip.h).

There is no CPU fallback: if the library is missing, or an entry point reports an error, the call
raises.
"""
from __future__ import annotations

import ctypes
import os
import threading
from typing import Optional

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libcrystalframer_hip.so")
ABI_VERSION = 13

CFH_WINDOW_REFERENCE = 0
CFH_WINDOW_WIDE = 1
FLAG_SINGLE_STREAM = 1      # cfh_params.flags: CFH_FLAG_SINGLE_STREAM
FLAG_DEFER_JOIN = 2         # cfh_params.flags: CFH_FLAG_DEFER_JOIN
FLAG_NO_WEIGHT_GRADS = 4    # cfh_params.flags: CFH_FLAG_NO_WEIGHT_GRADS


class CfhParams(ctypes.Structure):
    _fields_ = [
        ("struct_size", ctypes.c_int32),
        ("num_heads", ctypes.c_int32),
        ("head_dim", ctypes.c_int32),
        ("dist_bins", ctypes.c_int32),
        ("angle_bins", ctypes.c_int32),
        ("cos_abs", ctypes.c_int32),
        ("lattice_range", ctypes.c_int32),
        ("minimum_range", ctypes.c_int32),
        ("window_mode", ctypes.c_int32),
        ("dist_max", ctypes.c_float),
        ("dist_wscale", ctypes.c_float),
        ("angle_wscale", ctypes.c_float),
        ("dist_coef", ctypes.c_float),
        ("angle_coef", ctypes.c_float),
        ("cutoff_radius", ctypes.c_float),
        ("prune_log2", ctypes.c_float),
        ("symm_break_noise", ctypes.c_float),
        ("noise_seed", ctypes.c_uint64),
        ("grad_coef_quirk", ctypes.c_int32),
        ("collect_stats", ctypes.c_int32),
        ("noise_seed_dev", ctypes.c_void_p),
        ("noise_seed_advance", ctypes.c_int32),
        ("flags", ctypes.c_int32),
    ]


class CfhAttentionInputsGrad(ctypes.Structure):
    """cfh_attention_inputs_grad of the C header."""
    _fields_ = [("qkv", ctypes.c_void_p), ("lattice_w", ctypes.c_void_p), ("gauss_scale_dev", ctypes.c_void_p),
                ("gqs", ctypes.c_void_p), ("gk", ctypes.c_void_p), ("gv", ctypes.c_void_p), ("ga", ctypes.c_void_p),
                ("gqkv", ctypes.c_void_p), ("gw_partial", ctypes.c_void_p),
                ("c1", ctypes.c_float), ("lb", ctypes.c_float), ("c2", ctypes.c_float), ("q_scale", ctypes.c_float),
                ("H", ctypes.c_int32), ("reserved0", ctypes.c_int32)]


class CfhCoreCache(ctypes.Structure):
    """Mirror of ``cfh_core_cache`` in include/crystalframer_hip.h."""
    _fields_ = [("shift_table", ctypes.c_void_p), ("pair_near", ctypes.c_void_p), ("wcat", ctypes.c_void_p),
                ("records", ctypes.c_void_p),
                ("shift_table_ready", ctypes.c_int32), ("wcat_ready", ctypes.c_int32),
                ("records_ready", ctypes.c_int32), ("reserved0", ctypes.c_int32)]


class CfhLinearGradJob(ctypes.Structure):
    """Mirror of ``cfh_linear_grad_job`` in include/crystalframer_hip.h."""
    _fields_ = [("x", ctypes.c_void_p), ("dy", ctypes.c_void_p), ("dW", ctypes.c_void_p), ("db", ctypes.c_void_p),
                ("N", ctypes.c_int64), ("I", ctypes.c_int64), ("O", ctypes.c_int64), ("ldx", ctypes.c_int64),
                ("ldy", ctypes.c_int64)]


class CfhCoreWgradJob(ctypes.Structure):
    """Mirror of ``cfh_core_wgrad_job`` in include/crystalframer_hip.h."""
    _fields_ = [("gout", ctypes.c_void_p), ("hist", ctypes.c_void_p), ("N", ctypes.c_int64),
                ("gW_dist", ctypes.c_void_p), ("gW_axis1", ctypes.c_void_p), ("gW_axis2", ctypes.c_void_p),
                ("gW_axis3", ctypes.c_void_p)]


class CfhAdamWJob(ctypes.Structure):
    """Mirror of ``cfh_adamw_job`` in include/crystalframer_hip.h."""
    _fields_ = [("param", ctypes.c_void_p), ("grad", ctypes.c_void_p), ("exp_avg", ctypes.c_void_p),
                ("exp_avg_sq", ctypes.c_void_p), ("n", ctypes.c_int64)]


EXPORTS = ("cfh_abi_version", "cfh_last_error", "cfh_workspace_bytes", "cfh_frame_axis1",
           "cfh_frame_axis2", "cfh_frame_axes", "cfh_framed_pe_forward", "cfh_framed_pe_forward_static", "cfh_frame_axes_framed_pe_forward",
           "cfh_framed_pe_backward", "cfh_framed_pe_backward_pairwise",
           "cfh_fused_dpa_forward", "cfh_fused_dpa_backward", "cfh_pair_layout_check",
           "cfh_crystal_mean_forward", "cfh_crystal_mean_backward", "cfh_timing_enable", "cfh_timing_read",
           "cfh_crystal_geometry", "cfh_small_linear_forward", "cfh_small_linear_dx", "cfh_linear_weight_bias_grad", "cfh_linear_weight_bias_grad_batch", "cfh_linear_weight_bias_grad_batch_workspace_bytes", "cfh_attention_inputs_forward",
           "cfh_attention_inputs_backward", "cfh_layer_bridge_forward", "cfh_layer_bridge_backward",
           "cfh_second_stream_fork", "cfh_second_stream_get", "cfh_second_stream_join",
           "cfh_fused_core_workspace_bytes", "cfh_fused_core_hist_words", "cfh_fused_core_forward",
           "cfh_fused_core_backward", "cfh_adamw_step_batch",
           "cfh_fused_core_weight_gradients_workspace_bytes", "cfh_fused_core_weight_gradients")

_lib = None
_lock = threading.Lock()
_P = ctypes.c_void_p
_I64 = ctypes.c_int64


def load():
    """Load the library once; raise if it is absent or its ABI version differs."""
    global _lib
    if _lib is not None:
        return _lib
    with _lock:
        if _lib is not None:
            return _lib
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                f"{LIB_PATH} is missing: build it with `python -m crystalframer_amd.build` "
                "(hipcc --offload-arch=gfx950). There is no fallback path.")
        lib = ctypes.CDLL(LIB_PATH)
        for name in EXPORTS:
            if not hasattr(lib, name):
                raise RuntimeError(f"{LIB_PATH} does not export {name}")
        lib.cfh_abi_version.restype = ctypes.c_int
        lib.cfh_last_error.restype = ctypes.c_char_p
        lib.cfh_workspace_bytes.restype = ctypes.c_size_t
        lib.cfh_workspace_bytes.argtypes = [ctypes.POINTER(CfhParams), _I64, _I64]
        pp = ctypes.POINTER(CfhParams)
        lib.cfh_frame_axis1.restype = ctypes.c_int
        lib.cfh_frame_axis1.argtypes = [pp] + [_P] * 10 + [_I64] * 3 + [_P, _P, ctypes.c_size_t, _P]
        lib.cfh_frame_axis2.restype = ctypes.c_int
        lib.cfh_frame_axis2.argtypes = [pp] + [_P] * 11 + [_I64] * 3 + [_P, _P, ctypes.c_size_t, _P]
        lib.cfh_frame_axes.restype = ctypes.c_int
        lib.cfh_frame_axes.argtypes = [pp] + [_P] * 10 + [_I64] * 3 + [_P, _P, ctypes.c_size_t, _P]
        lib.cfh_framed_pe_forward.restype = ctypes.c_int
        lib.cfh_framed_pe_forward.argtypes = [pp] + [_P] * 13 + [_I64] * 3 + [_P] * 5 + [ctypes.c_size_t, _P]
        lib.cfh_framed_pe_forward_static.restype = ctypes.c_int
        lib.cfh_framed_pe_forward_static.argtypes = [pp] + [_P] * 13 + [_I64] * 3 + [_P] * 4 + [_P]
        lib.cfh_frame_axes_framed_pe_forward.restype = ctypes.c_int
        lib.cfh_frame_axes_framed_pe_forward.argtypes = [pp] + [_P] * 14 + [_I64] * 3 + [_P] * 6 + [ctypes.c_size_t, _P]
        lib.cfh_layer_bridge_forward.restype = ctypes.c_int
        lib.cfh_layer_bridge_forward.argtypes = ([_P, _P, _I64, ctypes.c_int32, ctypes.c_int32] + [_P] * 10
                                                 + [ctypes.c_float] * 4 + [ctypes.c_int32] + [_P] * 9)
        lib.cfh_layer_bridge_backward.restype = ctypes.c_int
        lib.cfh_layer_bridge_backward.argtypes = [_P] * 7 + [_I64, ctypes.c_int32, ctypes.c_int32] + [_P] * 6
        lib.cfh_framed_pe_backward.restype = ctypes.c_int
        lib.cfh_framed_pe_backward.argtypes = [pp] + [_P] * 17 + [_I64] * 3 + [_P] * 6 + [ctypes.c_size_t, _P]
        lib.cfh_framed_pe_backward_pairwise.restype = ctypes.c_int
        lib.cfh_framed_pe_backward_pairwise.argtypes = [pp] + [_P] * 12 + [_I64] * 3 + [_P, _P, ctypes.c_size_t, _P]
        lib.cfh_fused_dpa_forward.restype = ctypes.c_int
        lib.cfh_fused_dpa_forward.argtypes = [_P] * 7 + [_I64] * 4 + [_P] * 3
        lib.cfh_fused_dpa_backward.restype = ctypes.c_int
        lib.cfh_fused_dpa_backward.argtypes = [_P] * 10 + [_I64] * 4 + [_P] * 6
        lib.cfh_pair_layout_check.restype = ctypes.c_int
        lib.cfh_pair_layout_check.argtypes = [_P, _P, _I64, _I64, _P, _P]
        lib.cfh_crystal_mean_forward.restype = ctypes.c_int
        lib.cfh_crystal_mean_forward.argtypes = [_P, _P, _I64, _I64, _I64, _P, _P]
        lib.cfh_crystal_mean_backward.restype = ctypes.c_int
        lib.cfh_crystal_mean_backward.argtypes = [_P, _P, _P, _I64, _I64, _I64, _P, _P]
        lib.cfh_linear_weight_bias_grad.restype = ctypes.c_int
        lib.cfh_linear_weight_bias_grad.argtypes = [_P, _P, _I64, _I64, _I64, _P, _P, _P]
        lib.cfh_small_linear_forward.restype = ctypes.c_int
        lib.cfh_small_linear_forward.argtypes = [_P, _P, _P, _I64, _I64, _I64, ctypes.c_int32, _P, _P]
        lib.cfh_fused_core_weight_gradients_workspace_bytes.restype = ctypes.c_size_t
        lib.cfh_fused_core_weight_gradients_workspace_bytes.argtypes = [_P, ctypes.c_int32]
        lib.cfh_fused_core_weight_gradients.restype = ctypes.c_int
        lib.cfh_fused_core_weight_gradients.argtypes = [_P, _P, ctypes.c_int32, _P, ctypes.c_size_t, _P]
        lib.cfh_adamw_step_batch.restype = ctypes.c_int
        lib.cfh_adamw_step_batch.argtypes = [_P, ctypes.c_int32, ctypes.c_float, ctypes.c_float, ctypes.c_float,
                                             ctypes.c_float, ctypes.c_float, _P, _P]
        lib.cfh_small_linear_dx.restype = ctypes.c_int
        lib.cfh_small_linear_dx.argtypes = [_P, _P, _I64, _I64, _I64, _P, _P]
        lib.cfh_crystal_geometry.restype = ctypes.c_int
        lib.cfh_crystal_geometry.argtypes = [_P, _P, _P, _P, _I64, _I64, _I64] + [_P] * 8 + [_P, ctypes.c_size_t, _P]
        lib.cfh_linear_weight_bias_grad_batch.restype = ctypes.c_int
        lib.cfh_linear_weight_bias_grad_batch.argtypes = [ctypes.POINTER(CfhLinearGradJob), ctypes.c_int32, _P,
                                                          ctypes.c_size_t, _P]
        lib.cfh_linear_weight_bias_grad_batch_workspace_bytes.restype = ctypes.c_size_t
        lib.cfh_linear_weight_bias_grad_batch_workspace_bytes.argtypes = [ctypes.POINTER(CfhLinearGradJob),
                                                                          ctypes.c_int32]
        _F, _I32 = ctypes.c_float, ctypes.c_int32
        lib.cfh_attention_inputs_forward.restype = ctypes.c_int
        lib.cfh_attention_inputs_forward.argtypes = [_P, _P, _P, _F, _F, _F, _F, _I64, _I32, _I32, _P, _P, _P, _P, _P]
        lib.cfh_attention_inputs_backward.restype = ctypes.c_int
        lib.cfh_attention_inputs_backward.argtypes = [_P, _P, _P, _F, _F, _F, _F, _P, _P, _P, _P, _I64, _I32, _I32,
                                                      _P, _P, _P, ctypes.c_size_t, _P]
        lib.cfh_fused_core_workspace_bytes.restype = ctypes.c_size_t
        lib.cfh_fused_core_workspace_bytes.argtypes = [pp, _I64, _I64, _I64, ctypes.c_int32]
        lib.cfh_fused_core_hist_words.restype = ctypes.c_int32
        lib.cfh_fused_core_hist_words.argtypes = [pp]
        lib.cfh_fused_core_forward.restype = ctypes.c_int
        pc = ctypes.POINTER(CfhCoreCache)
        lib.cfh_fused_core_forward.argtypes = ([pp] + [_P] * 15 + [_I64] * 3 + [_P, ctypes.c_int32] + [_P] * 4
                                               + [pc, _P, ctypes.c_size_t, _P])
        lib.cfh_fused_core_backward.restype = ctypes.c_int
        lib.cfh_fused_core_backward.argtypes = ([pp] + [_P] * 21 + [_I64] * 3 + [_P] * 9
                                                + [pc, _P, ctypes.c_size_t, _P])
        lib.cfh_timing_enable.restype = ctypes.c_int
        lib.cfh_timing_enable.argtypes = [ctypes.c_int]
        lib.cfh_timing_read.restype = ctypes.c_int
        lib.cfh_timing_read.argtypes = [ctypes.c_char_p, ctypes.POINTER(ctypes.c_double), ctypes.POINTER(_I64)]
        lib.cfh_second_stream_fork.restype = ctypes.c_int
        lib.cfh_second_stream_fork.argtypes = [_P, ctypes.POINTER(_P)]
        lib.cfh_second_stream_get.restype = ctypes.c_int
        lib.cfh_second_stream_get.argtypes = [ctypes.POINTER(_P)]
        lib.cfh_second_stream_join.restype = ctypes.c_int
        lib.cfh_second_stream_join.argtypes = [_P]
        if lib.cfh_abi_version() != ABI_VERSION:
            raise RuntimeError(f"ABI version {lib.cfh_abi_version()} of {LIB_PATH} != {ABI_VERSION}")
        _lib = lib
    return _lib


def check(rc: int, what: str):
    if rc != 0:
        msg = load().cfh_last_error().decode("utf-8", "replace")
        raise RuntimeError(f"{what} failed (code {rc}): {msg}")


def ptr(t: Optional[torch.Tensor]):
    """Device pointer of a contiguous tensor (None -> NULL)."""
    if t is None:
        return None
    if not t.is_contiguous():
        raise ValueError("tensor passed to the HIP library must be contiguous")
    return ctypes.c_void_p(t.data_ptr())


def require_gpu(*tensors: torch.Tensor):
    for t in tensors:
        if t is not None and not t.is_cuda:
            raise RuntimeError(
                "crystalframer_amd operators run on a HIP device only (tensor on "
                f"{t.device}); there is no CPU path")


_workspaces = {}
_superseded = []      # outgrown workspaces, kept for captured graphs that still point at them


def workspace(device: torch.device, nbytes: int) -> torch.Tensor:
    """Scratch buffer handed to the library, one per (device, stream): kernels of one stream run
    in order, so they can share it; grown on demand, reused across calls."""
    key = (device.type, device.index, torch.cuda.current_stream(device).cuda_stream)
    buf = _workspaces.get(key)
    if buf is None or buf.numel() < nbytes:
        if buf is not None:
            # a HIP graph captured on this stream holds the address of the buffer it was given: a superseded
            # buffer stays allocated, so that replays keep writing into memory that is still theirs
            _superseded.append(buf)
        buf = torch.empty(max(nbytes, 1 << 20), dtype=torch.uint8, device=device)
        buf[:512].zero_()          # work-queue heads and the statistics block
        _workspaces[key] = buf
    return buf


_wgrad_scratch = {}


def wgrad_scratch(device: torch.device, stream_ptr, nbytes: int) -> torch.Tensor:
    """Scratch of cfh_linear_weight_bias_grad_batch for launches on ``stream_ptr`` (which need not be the framework's
    current stream, whose buffer ``workspace`` hands out): one buffer per (device, stream), grown on demand."""
    key = (device.type, device.index, int(getattr(stream_ptr, "value", stream_ptr) or 0))
    buf = _wgrad_scratch.get(key)
    if buf is None or buf.numel() < nbytes:
        if buf is not None:
            _superseded.append(buf)      # a captured graph may still hold its address
        buf = torch.empty(max(nbytes, 1 << 20), dtype=torch.uint8, device=device)
        _wgrad_scratch[key] = buf
    return buf


STAT_NAMES = ("fwd_evaluated", "fwd_in_box", "bwd_evaluated", "bwd_in_box", "frame1_scanned",
              "frame2_scanned", "fwd_pairs", "bwd_pairs", "fwd_visited")


def read_stats(device: torch.device, reset: bool = False) -> dict:
    """Term counts accumulated by launches made with ``collect_stats`` on this stream (synchronises)."""
    buf = workspace(device, 512)
    vals = buf[256:512].view(torch.int64).cpu().tolist()
    if reset:
        buf[256:512].zero_()
    out = dict(zip(STAT_NAMES, vals))
    if any(vals[16:24]):        # cycle counts of a diagnostics build (phase timing of the fused forward kernel)
        out["phase_cycles"] = vals[16:24]
    return out


def read_status(device: torch.device, reset: bool = False) -> int:
    """Status word of this stream's workspace (synchronises): 1 when a launch had to cut a translation box
    back to the largest half-width the kernels sum (32), i.e. where the result differs from the reference's
    box rule; 0 otherwise."""
    buf = workspace(device, 512)
    val = int(buf[16:20].view(torch.int32).cpu()[0])
    if reset:
        buf[16:20].zero_()
    return val


def current_stream_ptr(device: torch.device):
    return ctypes.c_void_p(torch.cuda.current_stream(device).cuda_stream)


def kernel_timing(enable: bool):
    """Switch the library's own HIP-event bracket around its lattice-sum kernels on or off."""
    check(load().cfh_timing_enable(1 if enable else 0), "cfh_timing_enable")


def read_kernel_timing(what: str):
    """(total milliseconds, launches) of the kernels recorded under ``what`` since the last read."""
    total, count = ctypes.c_double(0.0), _I64(0)
    check(load().cfh_timing_read(what.encode(), ctypes.byref(total), ctypes.byref(count)), "cfh_timing_read")
    return total.value, count.value
