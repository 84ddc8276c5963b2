"""MI355X-native (gfx950) implementation of CrystalFramer's periodic infinitely-connected attention.

``cuda_funcs`` holds the drop-in operator boundary (same autograd.Function names and signatures as
the reference's ``models/cuda_funcs``); the kernels live in ``csrc`` behind a C ABI
(``include/crystalframer_hip.h``).
"""
from . import _lib  # noqa: F401
from .cuda_funcs import (  # noqa: F401
    CUPY_AVAILABLE,
    ComputeFrame1MaximumMethodCUDA,
    ComputeFrame2MaximumMethodCUDA,
    ComputeFramesMaximumMethodCUDA,
    FusedDotProductAttentionCUDA,
    IrregularMeanCUDA,
    KernelManager,
    RealEncodingWithFramedProjFuncCUDA,
    compile_kernels,
)

__all__ = [
    "CUPY_AVAILABLE", "ComputeFrame1MaximumMethodCUDA", "ComputeFrame2MaximumMethodCUDA",
    "ComputeFramesMaximumMethodCUDA", "FusedDotProductAttentionCUDA", "IrregularMeanCUDA",
    "KernelManager", "RealEncodingWithFramedProjFuncCUDA", "compile_kernels",
]
