"""Crystal property regressor: atom embedding -> periodic-attention encoder -> pooling -> MLP.

Counterpart of ``Latticeformer`` (reference: models/latticeformer.py:32-287) for one GPU: same
sub-module names (``input_embeddings``, ``encoder``, ``mlp``), same initialisation.  The
single-process multi-GPU split of the reference (:209-273) is not part of this build.
"""
from __future__ import annotations

import copy

import torch
from torch import nn

from . import cuda_funcs
from .encoder import CrystalformerEncoderCUDA
from .params import LatticeformerParams, ModelParams

ATOM_FEAT_DIM = 98


def max_pool(x, batch, sizes):
    """Per-crystal maximum (reference: models/pooling.py:13-16, which splits by ``sizes``).  The crystal
    indices in ``batch`` need not start at 0 (the encoder accepts such batches as well)."""
    B = sizes.shape[0]
    out = torch.full((B,) + tuple(x.shape[1:]), -float("inf"), dtype=x.dtype, device=x.device)
    if batch.numel() == 0:
        return out
    idx = (batch - batch[0]).reshape((-1,) + (1,) * (x.dim() - 1)).expand_as(x)
    return out.scatter_reduce(0, idx, x, reduce="amax", include_self=True)


def avr_pool(x, batch, sizes):
    """Reference: models/pooling.py:19-25."""
    return cuda_funcs.IrregularMeanCUDA.apply(x, batch, sizes)


def _run_head(module: nn.Module, x: torch.Tensor) -> torch.Tensor:
    """``module(x)`` for the Identity / Linear / norm / ReLU stacks of the model's head, with every Linear
    (and a ReLU that follows it directly) going through ``cuda_funcs.linear``: same arithmetic, weight
    gradients in the batched launch, few-row products in the library's own kernel."""
    if not isinstance(module, nn.Sequential):
        return module(x)
    mods = [m for m in module if not isinstance(m, nn.Identity)]
    n = 0
    while n < len(mods):
        m = mods[n]
        if isinstance(m, nn.Linear) and x.is_cuda:
            fuse = n + 1 < len(mods) and isinstance(mods[n + 1], nn.ReLU)
            x = cuda_funcs.linear(x, m.weight, m.bias, relu=fuse)
            n += 2 if fuse else 1
        else:
            x = m(x)
            n += 1
    return x


class Latticeformer(nn.Module):
    def __init__(self, params: ModelParams = None):
        super().__init__()
        params = params if params is not None else ModelParams()
        self.params = params
        embedding_dim = copy.deepcopy(list(params.embedding_dim))
        num_layers, model_dim = params.num_layers, params.model_dim
        if params.use_cgcnn_feat or params.scale_grad > 0:
            raise NotImplementedError("use_cgcnn_feat / scale_grad are not implemented")
        lattice_params = LatticeformerParams().parseFromArgs(params)
        self.input_embeddings = nn.Linear(ATOM_FEAT_DIM, model_dim, bias=False)
        emb_scale = model_dim ** (-0.5)
        if params.t_fixup_init:
            emb_scale *= (9 * num_layers) ** (-1 / 4)
        nn.init.normal_(self.input_embeddings.weight, mean=0, std=emb_scale)
        self.encoder = CrystalformerEncoderCUDA(
            model_dim, params.head_num, activation=params.t_activation, num_encoder_layers=num_layers,
            dim_feedforward=params.ff_dim, dropout=params.dropout, t_fixup_init=params.t_fixup_init,
            no_layer_norm=params.t_fixup_init, lattice_params=lattice_params, k_dim=params.k_dim,
            v_dim=params.v_dim)
        norm = {"bn": nn.BatchNorm1d, "ln": nn.LayerNorm, "in": nn.InstanceNorm1d,
                "id": nn.Identity, "no": nn.Identity}.get(params.norm_type)
        if norm is None:
            raise NotImplementedError(f"norm_type: {params.norm_type}")
        dim_pooled = model_dim
        self.proj_before_pooling = nn.Identity()
        if params.pre_pooling_op == "w+bn+relu":
            dim_pooled = embedding_dim.pop(0)
            self.proj_before_pooling = nn.Sequential(nn.Linear(model_dim, dim_pooled), norm(dim_pooled), nn.ReLU(True))
        elif params.pre_pooling_op == "w+relu":
            dim_pooled = embedding_dim.pop(0)
            self.proj_before_pooling = nn.Sequential(nn.Linear(model_dim, dim_pooled), nn.ReLU(True))
        elif params.pre_pooling_op == "relu":
            self.proj_before_pooling = nn.ReLU(True)
        elif params.pre_pooling_op != "no":
            raise NotImplementedError(f"pre_pooling_op: {params.pre_pooling_op}")
        if params.pooling == "max":
            self.pooling_layer = max_pool
        elif params.pooling == "avr":
            self.pooling_layer = avr_pool
        else:
            raise NotImplementedError(f"pooling: {params.pooling}")
        final_dim = 1 if isinstance(params.targets, str) else len(params.targets)
        in_dim = [dim_pooled] + embedding_dim[:-1]
        layers = []
        for di, do in zip(in_dim, embedding_dim):
            layers += [nn.Linear(di, do), norm(do), nn.ReLU(True)]
        layers.append(nn.Linear(embedding_dim[-1], final_dim))
        self.mlp = nn.Sequential(*layers)

    def forward(self, data, this_epoch=None):
        """``data`` carries x (N,98), pos (N,3), batch (N), trans_vec (B,3,3), sizes (B)."""
        x = cuda_funcs.linear(data.x, self.input_embeddings.weight, self.input_embeddings.bias)
        num_pairs = getattr(data, "num_pairs", -1)
        x = self.encoder(x, data.pos, data.batch, data.trans_vec, data.sizes, this_epoch=this_epoch,
                         num_pairs=num_pairs if num_pairs is not None and num_pairs >= 0 else None,
                         batch_zero_based=bool(getattr(data, "zero_based", False)))
        x = _run_head(self.proj_before_pooling, x)
        x = self.pooling_layer(x, data.batch, data.sizes)
        return _run_head(self.mlp, x)


def load_reference_checkpoint(model: Latticeformer, state_dict, prefix: str = "swa_model.module.",
                              fold_target_statistics: bool = True) -> Latticeformer:
    """Load the weights of a checkpoint written by the reference's trainer into ``model``, the way the reference's
    demo does (demo.py:67-88): ``state_dict`` is the checkpoint's ``"state_dict"`` entry (read it with
    ``torch.load(path, weights_only=True)["state_dict"]``); the entries of the averaged model carry ``prefix``, which
    is stripped; the load is strict, i.e. every parameter name and shape must match (they are the reference's).
    With ``fold_target_statistics`` the checkpoint's ``target_std`` / ``target_mean`` are folded into the last linear
    layer so that the model predicts in the target's units."""
    own = {key[len(prefix):]: value for key, value in state_dict.items() if key.startswith(prefix)}
    if not own:
        raise KeyError(f"no entry of the checkpoint starts with {prefix!r}")
    model.load_state_dict(own)
    if fold_target_statistics and "target_std" in state_dict and "target_mean" in state_dict:
        last = model.mlp[-1]
        std = state_dict["target_std"].to(last.weight.device, last.weight.dtype)
        mean = state_dict["target_mean"].to(last.weight.device, last.weight.dtype)
        with torch.no_grad():
            last.weight.mul_(std[:, None])
            last.bias.mul_(std).add_(mean)
    return model
