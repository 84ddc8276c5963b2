"""Encoder stack around the periodic attention layer.

Counterpart of ``CrystalformerEncoderCUDA`` / ``CrystalformerEncoderLayerCUDA``
(reference: models/indexed_latticeformer_encoder.py:644-901): same sub-module and parameter names,
residual blocks without normalisation when T-Fixup is on, T-Fixup rescaling of the value / output /
feed-forward weights.  The per-batch geometry is prepared once on the device (``geometry.py``)
instead of in a Python loop over crystals.
"""
from __future__ import annotations

from typing import Callable, Optional, Union

import torch
import torch.nn.functional as F
from torch import Tensor, nn
from torch.nn.init import constant_, xavier_uniform_

from . import cuda_funcs, geometry
from .attention import CrystalformerMultiheadAttentionCUDA
from .params import LatticeformerParams


# Between the attention cores of consecutive layers everything acts on single atoms: one launch per layer
# (cuda_funcs.LayerBridgeHIP) when the layers have no layer norm, no active dropout and the ReLU activation.
FUSED_LAYER_BRIDGE = True


def _activation(name):
    if callable(name):
        return name
    if name == "relu":
        return F.relu
    if name == "gelu":
        return F.gelu
    raise RuntimeError(f"activation should be relu/gelu, not {name}")


class CrystalformerEncoderLayerCUDA(nn.Module):
    def __init__(self, d_model: int, nhead: int, dim_feedforward: int = 2048, dropout: float = 0.1,
                 activation: Union[str, Callable[[Tensor], Tensor]] = F.relu, layer_norm_eps: float = 1e-5,
                 norm_first: bool = False, no_layer_norm: bool = False,
                 params: Optional[LatticeformerParams] = None, k_dim: int = 0, v_dim: int = 0) -> None:
        super().__init__()
        params = params if params is not None else LatticeformerParams()
        self.domain = params.domain
        self.self_attn = CrystalformerMultiheadAttentionCUDA(d_model, nhead, dropout=dropout, kdim=k_dim,
                                                             vdim=v_dim, params=params)
        self.linear1 = nn.Linear(d_model, dim_feedforward)
        self.dropout = nn.Dropout(dropout) if dropout > 0 else nn.Identity()
        self.linear2 = nn.Linear(dim_feedforward, d_model)
        self.norm_first = norm_first
        self.norm1 = nn.LayerNorm(d_model, eps=layer_norm_eps) if not no_layer_norm else nn.Identity()
        self.norm2 = nn.LayerNorm(d_model, eps=layer_norm_eps) if not no_layer_norm else nn.Identity()
        self.dropout1 = nn.Dropout(dropout) if dropout > 0 else nn.Identity()
        self.dropout2 = nn.Dropout(dropout) if dropout > 0 else nn.Identity()
        self.activation = _activation(activation)
        xavier_uniform_(self.linear1.weight)
        xavier_uniform_(self.linear2.weight)
        constant_(self.linear1.bias, 0)
        constant_(self.linear2.bias, 0)

    def fixup_initialization(self, num_layers: int):
        """T-Fixup: scale four weight matrices by 0.67 * L^(-1/4)
        (reference: models/indexed_latticeformer_encoder.py:820-841)."""
        s = 0.67 * num_layers ** (-1.0 / 4.0)
        with torch.no_grad():
            for w in (self.linear1.weight, self.linear2.weight, self.self_attn.out_proj.weight,
                      self.self_attn.v_proj_weight):
                w.mul_(s)

    def _sa_block(self, x, batch, edges, pos_ij, dist2_min, trans, kr_base, rvecs, vcell, onehot, this_epoch):
        x = self.self_attn(x, x, x, batch, batch, edges, pos_ij, dist2_min, trans, kr_base, rvecs, vcell,
                           onehot, need_weights=False, this_epoch=this_epoch)[0]
        return self.dropout1(x)

    def _ff_block(self, x):
        if self.activation is F.relu:
            h = cuda_funcs.linear(x, self.linear1.weight, self.linear1.bias, relu=True)
        else:
            h = self.activation(cuda_funcs.linear(x, self.linear1.weight, self.linear1.bias))
        return self.dropout2(cuda_funcs.linear(self.dropout(h), self.linear2.weight, self.linear2.bias))

    def forward(self, src: Tensor, batch: Tensor, edges: Tensor, pos_ij: Tensor = None,
                dist2_min: Tensor = None, trans: Tensor = None, kr_base: Tensor = None,
                rvecs: Tensor = None, vcell: Tensor = None, onehot: Tensor = None,
                this_epoch: int = None) -> Tensor:
        x = src
        if self.norm_first:
            x = x + self._sa_block(self.norm1(x), batch, edges, pos_ij, dist2_min, trans, kr_base, rvecs,
                                   vcell, onehot, this_epoch)
            x = x + self._ff_block(self.norm2(x))
        else:
            x = self.norm1(x + self._sa_block(x, batch, edges, pos_ij, dist2_min, trans, kr_base, rvecs,
                                              vcell, onehot, this_epoch))
            x = self.norm2(x + self._ff_block(x))
        return x


class CrystalformerEncoderCUDA(nn.Module):
    def __init__(self, d_model: int = 512, nhead: int = 8, num_encoder_layers: int = 6,
                 dim_feedforward: int = 2048, dropout: float = 0.1,
                 activation: Union[str, Callable[[Tensor], Tensor]] = F.relu, layer_norm_eps: float = 1e-5,
                 norm_first: bool = False, t_fixup_init: bool = False, no_layer_norm: bool = False,
                 lattice_params: Optional[LatticeformerParams] = None, k_dim: int = 0, v_dim: int = 0) -> None:
        super().__init__()
        lattice_params = lattice_params if lattice_params is not None else LatticeformerParams()
        self.lattice_params = lattice_params
        self.layers = nn.ModuleList([
            CrystalformerEncoderLayerCUDA(d_model, nhead, dim_feedforward, dropout, activation, layer_norm_eps,
                                          norm_first, no_layer_norm,
                                          params=lattice_params.getLayerParameters(i), k_dim=k_dim, v_dim=v_dim)
            for i in range(num_encoder_layers)])
        if t_fixup_init:
            for layer in self.layers:
                layer.fixup_initialization(num_encoder_layers)
        self.num_layers = num_encoder_layers
        self.norm = nn.LayerNorm(d_model, eps=layer_norm_eps) if not no_layer_norm else None
        self.d_model = d_model
        self.nhead = nhead
        P = lattice_params
        cuda_funcs.compile_kernels(
            P.lattice_range, nhead, k_dim if k_dim > 0 else d_model // nhead, P.value_pe_dist_real,
            P.value_pe_angle_real, v_dim if v_dim > 0 else d_model // nhead, P.minimum_range, P.cos_abs,
            P.value_pe_dist_wscale, P.value_pe_angle_wscale, P.value_pe_dist_coef, P.value_pe_angle_coef,
            P.symm_break_noise)

    def _bridge_ready(self, x: Tensor) -> bool:
        if not (FUSED_LAYER_BRIDGE and x.is_cuda and x.dtype == torch.float32 and x.dim() == 2):
            return False
        for layer in self.layers:
            at = layer.self_attn
            idle = lambda m: isinstance(m, nn.Identity) or not self.training or getattr(m, "p", 0.0) == 0.0
            if not (isinstance(layer.norm1, nn.Identity) and isinstance(layer.norm2, nn.Identity)
                    and layer.activation is F.relu and idle(layer.dropout) and idle(layer.dropout1)
                    and idle(layer.dropout2) and at.fused_inputs_ready() and at.vdim == self.d_model
                    and cuda_funcs.LayerBridgeHIP.supported(self.d_model, layer.linear1.out_features, at.num_heads)
                    and layer.linear1.weight.dtype == torch.float32):
                return False
        return True

    def _forward_bridged(self, x: Tensor, batch: Tensor, geo, trans: Tensor, this_epoch) -> Tensor:
        """The layers as: input projection of the first, then per layer the attention core and ONE launch
        for all that follows it up to the next core (same arithmetic as the modules' own forward)."""
        layers = self.layers
        q, k, v, a = layers[0].self_attn.project_inputs(x)
        for n, layer in enumerate(layers):
            at = layer.self_attn
            core, _ = at.attention_core(q, k, v, a, batch, batch, geo.edges, geo.rpos, None, trans, geo.rvlen,
                                        this_epoch, True)
            if n + 1 < len(layers):
                stacked, in_bias, lw, gs, H, c1, lb, c2, q_scale, qkv_w = layers[n + 1].self_attn.bridge_arguments()
            else:
                stacked = in_bias = lw = gs = None
                H, (c1, lb, c2), q_scale, qkv_w = at.num_heads, at._gauss_constants(), 1.0, ()
            out = cuda_funcs.LayerBridgeHIP.apply(
                core, x, at.out_proj.weight, at.out_proj.bias, layer.linear1.weight, layer.linear1.bias,
                layer.linear2.weight, layer.linear2.bias, stacked, in_bias, lw, gs, H, c1, lb, c2, q_scale, *qkv_w)
            if n + 1 < len(layers):
                x, q, k, v, a = out
            else:
                x, = out
        return x

    def forward(self, src: Tensor, pos: Tensor, batch: Tensor, trans: Tensor, sizes: Tensor,
                onehot: Tensor = None, this_epoch: int = None, num_pairs: int = None,
                batch_zero_based: bool = False) -> Tensor:
        """Reference: models/indexed_latticeformer_encoder.py:699-742.  ``num_pairs`` (sum of
        sizes^2) may be given when the caller knows it on the host: the geometry then needs no
        device-to-host read, which also makes the whole forward pass capturable in a HIP graph.
        ``batch_zero_based``: the crystal indices are known to start at 0 (the reference subtracts batch[0])."""
        if src.size(-1) != self.d_model:
            raise RuntimeError("the feature number of src and tgt must be equal to d_model")
        if not batch_zero_based:           # the caller may know that the crystal indices start at 0
            batch = batch - batch[0]
        geo = geometry.crystal_geometry(pos, batch, trans, sizes, num_edges=num_pairs)
        cuda_funcs.seed_edge_schedule(geo.edges, geo.e_start, geo.order)
        cuda_funcs.declare_complete_blocks(geo.edges)
        cuda_funcs.declare_shift_tables(trans)
        if geo.atom_start is not None and sizes is not None:
            cuda_funcs.seed_atom_start(sizes, geo.atom_start)
        x = src
        if self._bridge_ready(x):
            x = self._forward_bridged(x, batch, geo, trans, this_epoch)
        else:
            for layer in self.layers:
                # rvecs: the lengths of the reciprocal vectors are all the layers use, computed once here
                x = layer(x, batch, geo.edges, geo.rpos, None, trans, None, geo.rvlen, geo.vcell, onehot, this_epoch)
        if self.norm is not None:
            x = self.norm(x)
        return x
