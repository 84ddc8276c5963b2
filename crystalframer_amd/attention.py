"""Periodic infinitely-connected multi-head attention layer (real-space, max-frame method).

Counterpart of ``CrystalformerMultiheadAttentionCUDA`` and
``crystalformer_multi_head_attention_forward_cuda`` of the reference
(models/indexed_lattice_multi_head_attention_cuda.py:737-996,998-1268): the same parameter names
and shapes (so a reference checkpoint's ``self_attn.*`` entries load), the same forward arithmetic,
and the same calls into the operator boundary (``cuda_funcs``).  Only what the "real" domain with
``frame_method`` "max" (or no angle encoding) needs is implemented; other settings raise.
"""
from __future__ import annotations

import math
from typing import Optional, Tuple

import torch
import torch.nn.functional as F
from torch import Tensor, nn
from torch.nn.init import constant_, normal_, xavier_uniform_

from . import cuda_funcs
from .params import LatticeformerParams


FUSED_FRAMES = True      # one launch for both axes + orthogonalisation (False: the reference's three steps)
FUSED_FRAMES_PE = True   # frame search and lattice sums in one library call (False: two calls, as the reference makes them)
FUSED_INPUTS = True      # q/k/v split, query scaling and Gaussian coefficient in one launch (False: framework ops)
FUSED_CORE = True        # frames, lattice sums and softmax attention in one library call with one histogram per
                         # (atom, head) (cuda_funcs.PeriodicAttentionCoreHIP); False: the reference's sequence of operators


def compute_frame_maximum_method_(q, k, v, alpha, pos, dist2_min, tvecs, batch, edges, proj, K: int,
                                  dist_max: float, wscale: float, frame_method: str, this_epoch=None,
                                  rvecs: Optional[Tensor] = None, cutoff: Optional[float] = None,
                                  q_is_scaled: bool = False):
    """Three orthonormal frame axes per (atom, head).  ``q_is_scaled``: the query already carries
    the 1/sqrt(Dh) that the reference applies here.
    Reference: models/indexed_lattice_multi_head_attention_cuda.py:435-493."""
    adap = ()
    if cutoff is not None:
        rvlen = rvecs if rvecs.dim() == 2 else torch.norm(rvecs, 2, dim=-1)
        adap = (rvlen, cutoff)
    if not q_is_scaled:
        q = q / math.sqrt(q.shape[-1])
    if frame_method != "max":
        raise NotImplementedError(f"frame_method={frame_method!r}: only 'max' is implemented")
    if FUSED_FRAMES:
        frames = cuda_funcs.ComputeFramesMaximumMethodCUDA.apply(
            q, k, v, alpha, pos, dist2_min, tvecs, batch, edges, K, dist_max, wscale, *adap)
        return frames[0], frames[1], frames[2]
    frame1 = cuda_funcs.ComputeFrame1MaximumMethodCUDA.apply(
        q, k, v, alpha, pos, dist2_min, tvecs, batch, edges, K, dist_max, wscale, *adap)
    frame2_max = cuda_funcs.ComputeFrame2MaximumMethodCUDA.apply(
        q, k, v, alpha, pos, dist2_min, tvecs, batch, edges, K, dist_max, wscale, frame1, *adap)
    dot = (frame1 * frame2_max).sum(-1, keepdim=True)
    frame2 = F.normalize(frame2_max - dot * frame1, dim=2)
    frame3 = torch.linalg.cross(frame1, frame2)
    return frame1, frame2, frame3


def compute_real_domain_attn_frame_proj(q, k, v, batch_q, batch_kv, edges, pos, dist2_min, tvecs, rvecs,
                                        pe_dist_proj, proj_angle1, proj_angle2, proj_angle3, alpha,
                                        params: LatticeformerParams, this_epoch=None, frame_sink=None,
                                        q_is_scaled: bool = False):
    """z (E,H) and psi (E,H,Dh) for one layer.
    Reference: models/indexed_lattice_multi_head_attention_cuda.py:589-734 (frame_method 'max')."""
    K = params.value_pe_dist_real
    dist_max = params.value_pe_dist_max
    if dist_max < 0:
        dist_max = (-dist_max) * params.scale_real
    wscale = params.value_pe_dist_wscale
    adap = ()
    if params.adaptive_cutoff_sigma < 0:
        adap = (rvecs, params.adaptive_cutoff_sigma)
    elif params.adaptive_cutoff_sigma > 0:
        adap = (rvecs, params.scale_real * params.gauss_lb_real ** (-0.5) * params.adaptive_cutoff_sigma)
    if params.frame_method != "max":
        raise NotImplementedError(f"frame_method={params.frame_method!r}: only 'max' is implemented")
    rvlen_args = ()
    if adap:
        rv = adap[0]
        rvlen_args = (rv if rv.dim() == 2 else torch.norm(rv, 2, dim=-1), adap[1])
    use_angle = proj_angle1 is not None and params.value_pe_angle_real > 0
    if use_angle and FUSED_FRAMES and FUSED_FRAMES_PE and pe_dist_proj is not None and K > 0:
        # frame search and lattice sums in one library call (they share the per-item records)
        qs = q if q_is_scaled else q / math.sqrt(q.shape[-1])
        z, psi, frames = cuda_funcs.RealEncodingWithMaxFramesFuncHIP.apply(
            qs, k, alpha, pos, dist2_min, tvecs, batch_q, edges, K, dist_max, wscale, pe_dist_proj,
            proj_angle1, proj_angle2, proj_angle3, params.value_pe_angle_real, params.value_pe_angle_wscale,
            params.cos_abs, params.value_pe_dist_coef, params.value_pe_angle_coef, *rvlen_args)
        if frame_sink is not None:
            frame_sink.append((frames[0], frames[1], frames[2]))
        return z, psi
    if use_angle:
        # the reference computes the frames even when the angle encoding is off; their only consumer
        # is the angle encoding, so they are skipped here in that case
        f1, f2, f3 = compute_frame_maximum_method_(
            q, k, None, alpha, pos, dist2_min, tvecs, batch_q, edges, pe_dist_proj, K, dist_max, wscale,
            params.frame_method, this_epoch, *rvlen_args, q_is_scaled=q_is_scaled)
    else:
        f1 = f2 = f3 = None
    if frame_sink is not None:
        frame_sink.append((f1, f2, f3))
    out = cuda_funcs.RealEncodingWithFramedProjFuncCUDA.apply(
        alpha, pos, dist2_min, tvecs, batch_q, edges, K, dist_max, wscale, pe_dist_proj,
        proj_angle1 if use_angle else None, proj_angle2 if use_angle else None,
        proj_angle3 if use_angle else None, f1, f2, f3, params.value_pe_angle_real,
        params.value_pe_angle_wscale, params.cos_abs, params.value_pe_dist_coef,
        params.value_pe_angle_coef, *rvlen_args)
    if len(out) == 1:
        return out[0], None
    return out


def _scaled_dot_product_attention(q, k, v, batch, batch_kv, edges, attn_weights=None, values=None,
                                  q_is_scaled: bool = False):
    """Reference: models/indexed_lattice_multi_head_attention_cuda.py:144-185."""
    if not q_is_scaled:
        q = q / math.sqrt(q.shape[-1])
    return cuda_funcs.FusedDotProductAttentionCUDA.apply(q, k, v, attn_weights, values, batch, edges)


class CrystalformerMultiheadAttentionCUDA(nn.Module):
    def __init__(self, embed_dim, num_heads, dropout=0.0, bias=True, kdim=None, vdim=None,
                 params: Optional[LatticeformerParams] = None, device=None, dtype=None) -> None:
        fk = {"device": device, "dtype": dtype}
        super().__init__()
        params = params if params is not None else LatticeformerParams()
        if params.domain != "real":
            raise NotImplementedError(f"domain={params.domain!r}: only the real-space domain is implemented")
        if not params.gauss_state.startswith("q"):
            raise NotImplementedError(f"gauss_state={params.gauss_state!r}: only 'q*' is implemented")
        if dropout != 0.0:
            raise NotImplementedError("attention dropout is not implemented (the reference default is 0)")
        self.embed_dim = embed_dim
        self.kdim = kdim * num_heads if kdim is not None and kdim > 0 else embed_dim
        self.vdim = vdim * num_heads if vdim is not None and vdim > 0 else embed_dim
        self.params = params
        self.gauss_scale = nn.Parameter(torch.zeros(2, **fk), requires_grad=False)
        self.atten_scale = nn.Parameter(torch.zeros(1, **fk), requires_grad=False)
        self.num_heads = num_heads
        self.dropout = dropout
        self.head_dim = embed_dim // num_heads
        assert self.head_dim * num_heads == embed_dim, "embed_dim must be divisible by num_heads"
        self.q_proj_weight = nn.Parameter(torch.empty((self.kdim, embed_dim), **fk))
        self.k_proj_weight = nn.Parameter(torch.empty((self.kdim, embed_dim), **fk))
        self.v_proj_weight = nn.Parameter(torch.empty((self.vdim, embed_dim), **fk))
        if bias:
            self.in_proj_bias = nn.Parameter(torch.empty(self.kdim * 2 + self.vdim, **fk))
        else:
            self.register_parameter("in_proj_bias", None)
        self.out_proj = nn.Linear(self.vdim, embed_dim, bias=bias, **fk)
        self.lattice_pos_weights = nn.Parameter(torch.empty((self.kdim,), **fk))
        H, Dh = num_heads, self.head_dim
        self.pe_dist_proj = nn.Parameter(torch.empty(1, H, Dh, params.value_pe_dist_real, **fk)) \
            if params.value_pe_dist_real > 0 else None
        self.pe_wave_proj = None
        if params.value_pe_wave_real > 0:
            raise NotImplementedError("value_pe_wave_real > 0 is not implemented")
        for n in (1, 2, 3):
            w = nn.Parameter(torch.empty(1, H, Dh, params.value_pe_angle_real, **fk)) \
                if params.value_pe_angle_real > 0 else None
            setattr(self, f"proj_angle{n}", w)
        self._gauss_ready = None      # host-side cache of "gauss_scale[0] > 0"
        self._in_proj_stack = None    # the storage q/k/v_proj_weight share once they are adjacent
        self.frame_sink = None        # a list: every forward appends its (f1, f2, f3) (diagnostics)
        self.grad_sink = None         # a dict: the backward pass leaves the gradients of the attention core's operands
                                      # (scaled query "q", "k", "v", Gaussian coefficient "a") in it (diagnostics)
        self._reset_parameters()

    def _reset_parameters(self):
        """Reference: models/indexed_lattice_multi_head_attention_cuda.py:1111-1196."""
        xavier_uniform_(self.q_proj_weight)
        xavier_uniform_(self.k_proj_weight)
        xavier_uniform_(self.v_proj_weight)
        xavier_uniform_(self.out_proj.weight)
        if self.in_proj_bias is not None:
            constant_(self.in_proj_bias, 0.0)
            constant_(self.out_proj.bias, 0.0)
        gs = self.params.gauss_state
        if gs in ("q", "q-headdim"):
            normal_(self.lattice_pos_weights, 0.0, (self.kdim // self.num_heads) ** -0.5)
        elif gs == "q-kdim":
            normal_(self.lattice_pos_weights, 0.0, self.kdim ** -0.5)
        else:
            raise NotImplementedError(gs)
        with torch.no_grad():
            for W in (self.pe_dist_proj, self.proj_angle1, self.proj_angle2, self.proj_angle3):
                if W is None:
                    continue
                for Wi in W:                      # (H, Dh, bins) viewed as (H*Dh, bins)
                    Wv = Wi.view(-1, Wi.shape[-1])
                    xavier_uniform_(Wv, Wv.shape[1] ** -0.5)

    def _load_from_state_dict(self, *args, **kwargs):
        self._gauss_ready = None
        return super()._load_from_state_dict(*args, **kwargs)

    def _stacked_in_proj(self) -> Tensor:
        """The three input-projection weights as one (2 kdim + vdim, E) matrix without a copy per step:
        the parameters live as adjacent row blocks of one storage.  Re-established here whenever
        something gave them storages of their own (``.to(device)``, ``load_state_dict(assign=True)``);
        values, names and shapes of the parameters do not change."""
        q, k, v = self.q_proj_weight, self.k_proj_weight, self.v_proj_weight
        st = self._in_proj_stack
        es = q.element_size()
        adjacent = (st is not None and st.device == q.device and st.dtype == q.dtype
                    and q.data_ptr() == st.data_ptr() and k.data_ptr() == q.data_ptr() + q.numel() * es
                    and v.data_ptr() == k.data_ptr() + k.numel() * es
                    and q.is_contiguous() and k.is_contiguous() and v.is_contiguous())
        if not adjacent:
            with torch.no_grad():
                st = torch.cat([q.data, k.data, v.data], dim=0)
                q.data = st[:q.shape[0]]
                k.data = st[q.shape[0]:q.shape[0] + k.shape[0]]
                v.data = st[q.shape[0] + k.shape[0]:]
            self._in_proj_stack = st
        return st

    def _gauss_constants(self):
        """(c1, lb, c2) of a = ((1 - lb) elu(c1 alpha') + 1) c2."""
        P = self.params
        lb = P.gauss_lb_real
        return P.positive_func_beta / (1.0 - lb), lb, -0.5 * P.scale_real ** -2

    def _gauss_scale_ready(self) -> bool:
        """True once gauss_scale holds the normalisation of alpha (one host read, then cached)."""
        if self._gauss_ready is None:
            self._gauss_ready = bool(self.gauss_scale[0] > 0)
        return self._gauss_ready

    def gaussian_coefficient(self, q: Tensor) -> Tensor:
        """alpha = q_h . w_h, normalised, mapped to a = [(1-lb) elu(alpha beta/(1-lb)) + 1] (-1/2 r0^-2).
        Reference: models/indexed_lattice_multi_head_attention_cuda.py:896-940."""
        P = self.params
        N, H, Dh = q.shape
        alpha = (q * self.lattice_pos_weights.view(1, H, Dh)).sum(-1)
        if P.normalize_gauss:
            if self._gauss_ready is None:
                self._gauss_ready = bool(self.gauss_scale[0] > 0)      # one host read, then cached
            if self._gauss_ready:
                scale, shift = self.gauss_scale[0], self.gauss_scale[1]
            else:
                scale = torch.reciprocal(alpha.detach().std())
                shift = -alpha.detach().mean()
                if self.training:
                    with torch.no_grad():
                        self.gauss_scale[0] = scale
                        self.gauss_scale[1] = shift
                    self._gauss_ready = True
            alpha = (alpha + shift) * scale
        lb, beta = P.gauss_lb_real, P.positive_func_beta
        return ((1.0 - lb) * F.elu(alpha * (beta / (1.0 - lb))) + 1.0) * (-0.5 * P.scale_real ** -2)

    def forward(self, query: Tensor, key: Tensor, value: Tensor, batch_q: Tensor, batch_kv: Tensor,
                edges: Tensor, points: Tensor, dist2_min: Optional[Tensor], tvecs: Tensor,
                kr_base: Optional[Tensor] = None, rvecs: Optional[Tensor] = None,
                vcell: Optional[Tensor] = None, onehot: Optional[Tensor] = None,
                need_weights: bool = False, this_epoch: Optional[int] = None) -> Tuple[Tensor, Optional[Tensor]]:
        """``points`` is rpos_ij (E,3) as in the reference's call
        (models/indexed_latticeformer_encoder.py:884); ``rvecs`` may be the reciprocal vectors
        (B,3,3) or their lengths (B,3).  Returns (attn_output (N,E), psi)."""
        if need_weights:
            raise NotImplementedError("need_weights=True is not implemented")
        N = query.shape[0]
        H, Dh = self.num_heads, self.head_dim
        q_is_scaled = False
        if self.in_proj_bias is None:
            bq = bk = bv = None
        else:
            bq, bk, bv = self.in_proj_bias.split([self.kdim, self.kdim, self.vdim])
        if query is key and key is value:
            # self-attention: the three projections as one GEMM over the stacked weights (same
            # arithmetic per output element; forward, input gradient and weight gradient each
            # become one launch instead of three)
            qkv = cuda_funcs.linear(query, (self.q_proj_weight, self.k_proj_weight, self.v_proj_weight),
                                    self.in_proj_bias, stacked=self._stacked_in_proj())
            fused = (FUSED_INPUTS and self.kdim == self.vdim == H * Dh
                     and cuda_funcs.AttentionInputsHIP.supported(H, Dh)
                     and (not self.params.normalize_gauss or self._gauss_scale_ready()))
            if fused:
                # split, query scaling and Gaussian coefficient in one launch (one more in backward)
                c1, lb, c2 = self._gauss_constants()
                q, k, v, a = cuda_funcs.AttentionInputsHIP.apply(
                    qkv, self.lattice_pos_weights, self.gauss_scale if self.params.normalize_gauss else None,
                    H, c1, lb, c2, 1.0 / math.sqrt(Dh))
                q_is_scaled = True
            else:
                q, k, v = qkv.split([self.kdim, self.kdim, self.vdim], dim=1)
                q = q.reshape(N, H, -1)
                k = k.reshape(N, H, -1)
                v = v.reshape(N, H, -1)
        else:
            q = cuda_funcs.linear(query, self.q_proj_weight, bq).view(N, H, -1)
            k = cuda_funcs.linear(key, self.k_proj_weight, bk).view(key.shape[0], H, -1)
            v = cuda_funcs.linear(value, self.v_proj_weight, bv).view(value.shape[0], H, -1)
        if not q_is_scaled:
            a = self.gaussian_coefficient(q)
        out, psi = self.attention_core(q, k, v, a, batch_q, batch_kv, edges, points, dist2_min, tvecs, rvecs,
                                       this_epoch, q_is_scaled)
        out = cuda_funcs.linear(out, self.out_proj.weight, self.out_proj.bias)
        return out, psi

    def attention_core(self, q: Tensor, k: Tensor, v: Tensor, a: Tensor, batch_q: Tensor, batch_kv: Tensor,
                       edges: Tensor, points: Tensor, dist2_min: Optional[Tensor], tvecs: Tensor,
                       rvecs: Optional[Tensor], this_epoch: Optional[int], q_is_scaled: bool):
        """Frames, lattice sums and the softmax attention for projected q, k, v (N,H,Dh) and Gaussian
        coefficients a (N,H): the heads' outputs side by side (N, H Dv), before the output projection,
        and psi."""
        P = self.params
        if not q_is_scaled:
            q, q_is_scaled = q / math.sqrt(q.shape[-1]), True
        if self.grad_sink is not None:
            for name, t in (("q", q), ("k", k), ("v", v), ("a", a)):
                if t.requires_grad:
                    t.register_hook(lambda grad, name=name: self.grad_sink.__setitem__(name, grad.detach()))
        if (FUSED_CORE and q.is_cuda and P.frame_method == "max" and batch_q is batch_kv and self.pe_dist_proj is not None
                and cuda_funcs.PeriodicAttentionCoreHIP.supported(
                    P.value_pe_dist_real, P.value_pe_angle_real, P.value_pe_dist_wscale, P.value_pe_angle_wscale,
                    self.pe_dist_proj, self.proj_angle1)):
            # one library call: frame search, lattice sums, softmax over the pairs, value encoding through one
            # histogram per (atom, head); psi is never formed
            dist_max = P.value_pe_dist_max if P.value_pe_dist_max >= 0 else -P.value_pe_dist_max * P.scale_real
            rvlen = cutoff = None
            if P.adaptive_cutoff_sigma != 0:
                rvlen = rvecs if rvecs.dim() == 2 else torch.norm(rvecs, 2, dim=-1)
                cutoff = (P.adaptive_cutoff_sigma if P.adaptive_cutoff_sigma < 0
                          else P.scale_real * P.gauss_lb_real ** (-0.5) * P.adaptive_cutoff_sigma)
            qs = q if q_is_scaled else q / math.sqrt(q.shape[-1])
            use_angle = self.proj_angle1 is not None and P.value_pe_angle_real > 0
            out, frames = cuda_funcs.PeriodicAttentionCoreHIP.apply(
                qs, k, v, a, points, tvecs, batch_q, edges, P.value_pe_dist_real, dist_max, P.value_pe_dist_wscale,
                self.pe_dist_proj, self.proj_angle1 if use_angle else None, self.proj_angle2 if use_angle else None,
                self.proj_angle3 if use_angle else None, P.value_pe_angle_real, P.value_pe_angle_wscale, P.cos_abs,
                P.value_pe_dist_coef, P.value_pe_angle_coef, rvlen, cutoff, None)
            if self.frame_sink is not None:
                self.frame_sink.append((None, None, None) if frames is None else (frames[0], frames[1], frames[2]))
            return out.reshape(q.shape[0], self.num_heads * v.shape[-1]), None
        z, psi = compute_real_domain_attn_frame_proj(
            q, k, v, batch_q, batch_kv, edges, points, dist2_min, tvecs, rvecs, self.pe_dist_proj,
            self.proj_angle1, self.proj_angle2, self.proj_angle3, a, self.params, this_epoch,
            frame_sink=self.frame_sink, q_is_scaled=q_is_scaled)
        out = _scaled_dot_product_attention(q, k, v, batch_q, batch_kv, edges, z, psi, q_is_scaled=q_is_scaled)
        return out.reshape(q.shape[0], self.num_heads * v.shape[-1]), psi

    def fused_inputs_ready(self) -> bool:
        """True when the input projection can be followed by the fused split / scaling / Gaussian
        coefficient (AttentionInputsHIP, or the last stage of LayerBridgeHIP)."""
        H, Dh = self.num_heads, self.head_dim
        return (FUSED_INPUTS and self.kdim == self.vdim == H * Dh
                and cuda_funcs.AttentionInputsHIP.supported(H, Dh)
                and (not self.params.normalize_gauss or self._gauss_scale_ready()))

    def bridge_arguments(self):
        """What LayerBridgeHIP needs of this layer as the NEXT one: (stacked weight, in_proj_bias,
        lattice_pos_weights, gauss_scale or None, H, c1, lb, c2, q_scale, (q, k, v weights))."""
        c1, lb, c2 = self._gauss_constants()
        return (self._stacked_in_proj(), self.in_proj_bias, self.lattice_pos_weights,
                self.gauss_scale if self.params.normalize_gauss else None, self.num_heads, c1, lb, c2,
                1.0 / math.sqrt(self.head_dim), (self.q_proj_weight, self.k_proj_weight, self.v_proj_weight))

    def project_inputs(self, x: Tensor):
        """(qs, k, v, a) of self-attention on x with the fused path (requires fused_inputs_ready())."""
        H, Dh = self.num_heads, self.head_dim
        qkv = cuda_funcs.linear(x, (self.q_proj_weight, self.k_proj_weight, self.v_proj_weight),
                                self.in_proj_bias, stacked=self._stacked_in_proj())
        c1, lb, c2 = self._gauss_constants()
        return cuda_funcs.AttentionInputsHIP.apply(
            qkv, self.lattice_pos_weights, self.gauss_scale if self.params.normalize_gauss else None,
            H, c1, lb, c2, 1.0 / math.sqrt(Dh))
