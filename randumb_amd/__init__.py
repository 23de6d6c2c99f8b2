"""randumb_amd: MI355X (gfx950) implementation of RANDUMB's pseudorandom-matrix hot path.

Python surface mirroring the reference package ``rten_cpp`` (Clyde013/randumb) over hand-written HIP kernels
reached through the C ABI of ``librandumb_hip.so``.
"""
from . import _lib, hip, ops  # noqa: F401
from .RandumbTensor import CreateRandumbTensor, RandumbTensor, RandumbTensorConstructor, rt_mm  # noqa: F401
from .SillyLayers import (SillyConv2d, SillyEmbedding, SillyLinear, SillyModuleMixin, init_coef_normal, init_kaiming_uniform,  # noqa: F401
                          init_zeros, listgen, stepgen)

__all__ = [
    "CreateRandumbTensor", "RandumbTensor", "RandumbTensorConstructor", "rt_mm", "SillyLinear", "SillyConv2d", "SillyEmbedding",
    "SillyModuleMixin", "init_kaiming_uniform", "init_coef_normal", "init_zeros", "stepgen", "listgen", "ops", "hip",
]
