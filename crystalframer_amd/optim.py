"""AdamW over the library's batched update kernel.

The reference trains with ``torch.optim.AdamW`` (models/regression.py:298-301).  The update rule here is the same
(decoupled weight decay, bias-corrected moments; no amsgrad, no maximize); what differs is the launch: one library
kernel for all parameter tensors of a group (``cfh_adamw_step_batch``) instead of the framework's multi-tensor
machinery, which for a model of many small tensors is bound by its bookkeeping.  The step count lives on the device,
so a captured step keeps counting from replay to replay; ``lr`` and the other scalars are read on the host when
``step`` is called (a captured step replays the values of its capture: a learning-rate scheduler, as the
reference's trainer uses, needs the step captured again, or run eagerly, whenever it changes ``lr``).  The step
count is one word per parameter GROUP, not per parameter as in torch.optim.AdamW: all parameters of a group take
their first step together (a parameter that gets its first gradient later is bias-corrected with the group's count).
"""
import ctypes

import torch

from . import _lib


class AdamW(torch.optim.Optimizer):
    def __init__(self, params, lr=1e-3, betas=(0.9, 0.999), eps=1e-8, weight_decay=1e-2):
        if lr < 0.0 or eps < 0.0 or weight_decay < 0.0:
            raise ValueError("lr, eps and weight_decay must not be negative")
        if not (0.0 <= betas[0] < 1.0 and 0.0 <= betas[1] < 1.0):
            raise ValueError(f"betas {betas} must lie in [0, 1)")
        super().__init__(params, dict(lr=lr, betas=betas, eps=eps, weight_decay=weight_decay))
        self._flat = {}

    def _group_state(self, group):
        """Moments of all parameters of a group in two flat buffers and the step word; ``self.state[p]`` holds the
        parameter's views of them under torch.optim.AdamW's names, so that ``state_dict()`` saves them."""
        st = self._flat.setdefault(id(group), {})
        if not st:
            ps = [p for p in group["params"] if p.requires_grad]
            if not ps:
                return None
            dev = ps[0].device
            for p in ps:
                if p.dtype != torch.float32 or not p.is_cuda or p.device != dev:
                    raise RuntimeError("AdamW of crystalframer_amd needs float32 parameters on one HIP device")
            offs, total = [], 0
            for p in ps:
                offs.append(total)
                total += (p.numel() + 3) & ~3          # every view 16-byte aligned
            st["exp_avg"] = torch.zeros(total, dtype=torch.float32, device=dev)
            st["exp_avg_sq"] = torch.zeros(total, dtype=torch.float32, device=dev)
            st["step"] = torch.zeros(1, dtype=torch.int64, device=dev)
            st["offset"] = {id(p): o for p, o in zip(ps, offs)}
            for p, o in zip(ps, offs):
                self.state[p] = dict(step=st["step"], exp_avg=st["exp_avg"][o:o + p.numel()].view_as(p),
                                     exp_avg_sq=st["exp_avg_sq"][o:o + p.numel()].view_as(p))
        return st

    def load_state_dict(self, state_dict):
        """Loads like torch.optim.AdamW, then moves the loaded moments into the flat buffers."""
        super().load_state_dict(state_dict)
        loaded = {p: dict(s) for p, s in self.state.items()}
        self._flat = {}
        for group in self.param_groups:
            st = self._group_state(group)
            if st is None:
                continue
            for p in group["params"]:
                old = loaded.get(p)
                if old is None or not p.requires_grad:
                    continue
                self.state[p]["exp_avg"].copy_(old["exp_avg"])
                self.state[p]["exp_avg_sq"].copy_(old["exp_avg_sq"])
                st["step"].fill_(int(old["step"]))

    @torch.no_grad()
    def step(self, closure=None):
        loss = None
        if closure is not None:
            with torch.enable_grad():
                loss = closure()
        lib = _lib.load()
        for group in self.param_groups:
            st = self._group_state(group)
            if st is None:
                continue
            jobs = []
            for p in group["params"]:
                g = p.grad
                if g is None:
                    continue
                if g.is_sparse:
                    raise RuntimeError("sparse gradients are not supported")
                if not p.is_contiguous():
                    raise RuntimeError("AdamW of crystalframer_amd needs contiguous parameters")
                if not g.is_contiguous():
                    g = g.contiguous()
                o = st["offset"][id(p)]
                jobs.append((p, g, o))
            if not jobs:
                continue
            dev = jobs[0][0].device
            arr = (_lib.CfhAdamWJob * len(jobs))()
            m0, v0 = st["exp_avg"].data_ptr(), st["exp_avg_sq"].data_ptr()
            for a, (p, g, o) in zip(arr, jobs):
                a.param, a.grad = p.data_ptr(), g.data_ptr()
                a.exp_avg, a.exp_avg_sq, a.n = m0 + 4 * o, v0 + 4 * o, p.numel()
            b1, b2 = group["betas"]
            with torch.cuda.device(dev):
                rc = lib.cfh_adamw_step_batch(arr, len(jobs), float(group["lr"]), float(b1), float(b2),
                                              float(group["eps"]), float(group["weight_decay"]),
                                              _lib.ptr(st["step"]), _lib.current_stream_ptr(dev))
            _lib.check(rc, "cfh_adamw_step_batch")
            del jobs      # the gradients stay alive through p.grad (or, made contiguous here, through the stream order)
        return loss
