"""Hyper-parameters of the lattice attention, with the reference's field names and defaults.

Counterpart of models/latticeformer_params.py:5-87 of the reference (class ``LatticeformerParams``);
the training-level keys that accompany them in params/crystalframer/default_jarvis.json are kept in
``ModelParams`` below.
"""
from __future__ import annotations

import copy
from dataclasses import dataclass, field
from typing import List, Union


class LatticeformerParams:
    def __init__(self,
                 domain: str = "real",
                 lattice_range: int = 4,
                 minimum_range: bool = True,
                 adaptive_cutoff_sigma: float = -3.5,
                 gauss_lb_real: float = 0.5,
                 gauss_lb_reci: float = 0.5,
                 scale_real: Union[float, List[float]] = (1.4,),
                 scale_reci: Union[float, List[float]] = (2.2,),
                 normalize_gauss: bool = True,
                 value_pe_dist_real: int = 64,
                 value_pe_dist_coef: float = 1.0,
                 value_pe_dist_max: float = -10.0,
                 value_pe_dist_wscale: float = 1.0,
                 value_pe_wave_real: int = 0,
                 value_pe_dist_reci: int = 0,
                 value_pe_wave_reci: int = 0,
                 value_pe_angle_real: int = 16,
                 value_pe_angle_coef: float = 1.0,
                 value_pe_angle_wscale: float = 4.0,
                 positive_func_beta: float = 0.1,
                 layer_index: int = -1,
                 gauss_state: str = "q",
                 frame_method: str = "max",
                 frame_mode: str = "both",
                 cos_abs: int = 1,
                 symm_break_noise: float = 1e-5) -> None:
        self.layer_index = layer_index
        self.domain = domain
        self.cos_abs = cos_abs
        self.lattice_range = lattice_range
        self.minimum_range = minimum_range
        self.adaptive_cutoff_sigma = adaptive_cutoff_sigma
        self.gauss_lb_real = gauss_lb_real
        self.gauss_lb_reci = gauss_lb_reci
        self.scale_real = list(scale_real) if isinstance(scale_real, (list, tuple)) else scale_real
        self.scale_reci = list(scale_reci) if isinstance(scale_reci, (list, tuple)) else scale_reci
        self.normalize_gauss = normalize_gauss
        self.value_pe_dist_real = value_pe_dist_real
        self.value_pe_dist_coef = value_pe_dist_coef
        self.value_pe_dist_max = value_pe_dist_max
        self.value_pe_dist_wscale = value_pe_dist_wscale
        self.value_pe_wave_real = value_pe_wave_real
        self.value_pe_dist_reci = value_pe_dist_reci
        self.value_pe_wave_reci = value_pe_wave_reci
        self.value_pe_angle_real = value_pe_angle_real
        self.value_pe_angle_coef = value_pe_angle_coef
        self.value_pe_angle_wscale = value_pe_angle_wscale
        self.positive_func_beta = positive_func_beta
        self.gauss_state = gauss_state
        self.frame_mode = frame_mode
        self.frame_method = frame_method
        self.symm_break_noise = symm_break_noise

    def parseFromArgs(self, args):
        """Copy every attribute of ``args`` whose name matches one of ours."""
        for key in self.__dict__:
            self.__dict__[key] = getattr(args, key, self.__dict__[key])
        return self

    def getLayerParameters(self, layer_index: int) -> "LatticeformerParams":
        """Per-layer copy: list-valued scales are indexed cyclically by layer."""
        if self.domain in ("real", "reci", "multihead"):
            domain = self.domain
        else:
            parts = self.domain.split("-")
            domain = parts[layer_index % len(parts)]
        scale_real, scale_reci = self.scale_real, self.scale_reci
        if isinstance(scale_real, (list, tuple)):
            scale_real = scale_real[layer_index % len(scale_real)]
        if isinstance(scale_reci, (list, tuple)):
            scale_reci = scale_reci[layer_index % len(scale_reci)]
        p = copy.deepcopy(self)
        p.domain, p.scale_real, p.scale_reci, p.layer_index = domain, scale_real, scale_reci, layer_index
        return p

    def __repr__(self):
        return "LatticeformerParams(" + ", ".join(f"{k}={v!r}" for k, v in self.__dict__.items()) + ")"


@dataclass
class ModelParams:
    """Model-level keys of params/crystalframer/default_jarvis.json (the CrystalFramer defaults)."""
    num_layers: int = 4
    model_dim: int = 128
    ff_dim: int = 512
    head_num: int = 8
    k_dim: int = 0
    v_dim: int = 0
    t_fixup_init: bool = True
    embedding_dim: List[int] = field(default_factory=lambda: [128])
    t_activation: str = "relu"
    dropout: float = 0.0
    pooling: str = "avr"
    pre_pooling_op: str = "no"
    norm_type: str = "no"
    targets: Union[str, List[str]] = "e_form"
    use_cgcnn_feat: bool = False
    scale_grad: float = 0.0
    # lattice attention (defaults of the JSON, which differ from the class defaults above)
    domain: str = "real"
    lattice_range: int = 2
    minimum_range: bool = True
    adaptive_cutoff_sigma: float = -3.5
    gauss_lb_real: float = 0.5
    gauss_lb_reci: float = 0.5
    gauss_state: str = "q"
    normalize_gauss: bool = True
    positive_func_beta: float = 0.1
    scale_real: List[float] = field(default_factory=lambda: [1.4])
    scale_reci: List[float] = field(default_factory=lambda: [2.2])
    value_pe_dist_real: int = 64
    value_pe_dist_reci: int = 0
    value_pe_dist_coef: float = 1.0
    value_pe_wave_real: int = 0
    value_pe_wave_reci: int = 0
    value_pe_dist_max: float = -10.0
    value_pe_dist_wscale: float = 1.0
    frame_method: str = "max"
    cos_abs: int = 0
    value_pe_angle_real: int = 64
    value_pe_angle_wscale: float = 4.0
    value_pe_angle_coef: float = 1.0
    symm_break_noise: float = 1e-5
