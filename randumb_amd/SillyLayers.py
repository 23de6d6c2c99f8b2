"""Layers whose weights are ``RandumbTensor`` buffers and whose parameters are the coefficient tensors.

Mirrors the reference's layer module (src/rten_cpp/SillyLayers.py): ``stepgen`` / ``listgen`` seed generators, the
``init_*`` schemes with the coefficient variance scaling ``var(coef) = 3 * std^2 / k``, ``SillyModuleMixin``,
``SillyLinear`` and ``SillyEmbedding``.  Additive: ``SillyLinear(matrix_coef=True)`` gives every output row its own
coefficient vector (coef is ``(out_features, k)``), and ``fused=True`` (the default for matrix-coef) routes the
forward and both backward products through the fused kernels that never write the weight to memory.
"""
from __future__ import annotations

import math
import warnings
from types import GeneratorType
from typing import Optional, Union

import torch
import torch.nn as nn
import torch.nn.functional as F
from torch import Generator
from torch.nn.init import _calculate_correct_fan, calculate_gain

from . import ops
from .RandumbTensor import CreateRandumbTensor, RandumbTensor


def stepgen(offset, step):
    """offset, offset + step, offset + 2*step, ...: a whole model's seeds as two numbers (SillyLayers.py:25-29)."""
    i = 0
    while True:
        yield offset + step * i
        i += 1


def listgen(lst):
    """Seeds / coefficient dims taken from an explicit list (SillyLayers.py:32-34)."""
    for i in lst:
        yield i


def _target_std(weight: RandumbTensor, a: float, mode: str, nonlinearity: str) -> float:
    fan = _calculate_correct_fan(weight, mode)
    return calculate_gain(nonlinearity, a) / math.sqrt(fan)


def init_kaiming_uniform(weight: RandumbTensor, bias: Optional[RandumbTensor], seed: int, a: float = math.sqrt(5),
                         mode: str = "fan_in", nonlinearity: str = "leaky_relu", generator: Optional[Generator] = None) -> None:
    """Uniform coefficients scaled so the materialised weight has the std ``kaiming_uniform_`` would give it.

    Noise entries are U[-1, 1] (variance 1/3), so a weight entry ``sum_m noise * coef[m]`` has variance
    ``k * var(coef) / 3``; asking for ``out_std^2`` gives ``var(coef) = 3 * out_std^2 / k``
    (SillyLayers.py:62-71).  The bias uses the weight's fan-in and its own ``k`` (SillyLayers.py:74-79).
    """
    if generator is None:
        generator = torch.Generator(device=weight._coef.device).manual_seed(seed)
    if 0 in weight._coef.shape:
        warnings.warn("Initializing zero-element tensors is a no-op")
        return
    out_std = _target_std(weight, a, mode, nonlinearity)
    coef_std = math.sqrt(3 / weight.int_dim) * out_std
    bound = math.sqrt(3.0) * coef_std
    with torch.no_grad():
        weight._coef.uniform_(-bound, bound, generator=generator)
    if bias is not None:
        bias_std = math.sqrt(3 / bias.int_dim) * out_std
        bound = math.sqrt(3.0) * bias_std
        with torch.no_grad():
            bias._coef.uniform_(-bound, bound, generator=generator)


def init_coef_normal(weight: RandumbTensor, std: float, seed: int, generator: Optional[Generator] = None) -> None:
    """Normal coefficients with ``var(coef) = 3 * std^2 / k`` so the materialised weight has standard deviation ``std``."""
    if generator is None:
        generator = torch.Generator(device=weight._coef.device).manual_seed(seed)
    with torch.no_grad():
        weight._coef.normal_(0.0, math.sqrt(3.0 / weight.int_dim) * std, generator=generator)


def init_zeros(weight: RandumbTensor, bias: Optional[RandumbTensor]) -> None:
    with torch.no_grad():
        weight._coef.zero_()
        if bias is not None:
            bias._coef.zero_()


class SillyModuleMixin(nn.Module):
    """Shared overrides: rebuild the tensor buffers when the module is moved or cast, and the scale-bias inits."""

    def _apply(self, fn, recurse=True):
        # Parameters are converted first (nn.Module._apply), so a rebuilt tensor picks up its coefficient's new device
        # and dtype; a wrapper subclass cannot change device in place (SillyLayers.py:94-114).
        def wrapped_fn(inp):
            if isinstance(inp, RandumbTensor):
                return CreateRandumbTensor(inp._coef, inp.seed, inp.shape, inp.scale_bias, inp.fused_bias)
            return fn(inp)

        super()._apply(wrapped_fn)
        for name, buf in list(self._buffers.items()):
            if isinstance(buf, RandumbTensor):  # re-point at the parameter objects that now live on the module
                coef = getattr(self, f"{name}_coef", buf._coef)
                sb = getattr(self, f"{name}_scale_bias", buf.scale_bias)
                self._buffers[name] = CreateRandumbTensor(coef, buf.seed, buf.shape, sb, buf.fused_bias)
        return self

    def init_rt_scale_bias(self, val=0):
        for name, buf in list(self.named_buffers(recurse=False)):
            if isinstance(buf, RandumbTensor):
                sb = nn.Parameter(torch.tensor([val], dtype=buf.dtype, device=buf.device))
                self.register_parameter(f"{name}_scale_bias", sb)
                self._buffers[name] = CreateRandumbTensor(buf._coef, buf.seed, buf.shape, sb, buf.fused_bias)

    def init_zero_coef_uniform_bias(self):
        """Zero coefficients; the fused random bias, scaled by ``sqrt(3) * std``, carries the initial weight
        (SillyLayers.py:122-133)."""
        std = _target_std(self.weight, math.sqrt(5), "fan_in", "leaky_relu")
        self.init_rt_scale_bias(math.sqrt(3.0) * std)
        init_zeros(self.weight, self.bias)

    def init_uniform_coef_zero_bias(self):
        """Scaled uniform coefficients, scale-bias zero (SillyLayers.py:135-138)."""
        self.init_rt_scale_bias(0)
        init_kaiming_uniform(self.weight, self.bias, self.seed[0])


def _take(src, n):
    return [next(src) for _ in range(n)] if isinstance(src, GeneratorType) else src


class SillyLinear(SillyModuleMixin, nn.Module):
    """``y = x A^T + b`` with ``A`` (and ``b``) pseudorandom tensors.  Same constructor as the reference
    (SillyLayers.py:142-227): ``int_dim`` and ``seed`` are lists or generators yielding two values (weight, bias).

    Parameters: ``weight_coef`` (``(k,)`` or, with ``matrix_coef``, ``(out_features, k)``), ``bias_coef``,
    ``weight_scale_bias`` / ``bias_scale_bias``.  Buffers: ``weight``, ``bias``.
    """

    __constants__ = ["in_features", "out_features", "int_dim"]
    num_seeds = 2

    def __init__(self, in_features: int, out_features: int, int_dim: Union[list, GeneratorType], seed: Union[list, GeneratorType],
                 bias: bool = True, rt_bias: bool = False, device=None, dtype=None, matrix_coef: bool = False,
                 fused: Optional[bool] = None) -> None:
        super().__init__()
        self.in_features = in_features
        self.out_features = out_features
        self.rt_bias = rt_bias
        self.matrix_coef = matrix_coef
        self.fused = matrix_coef if fused is None else fused
        self.int_dim = _take(int_dim, self.num_seeds)
        self.seed = _take(seed, self.num_seeds)

        coef_shape = (out_features, self.int_dim[0]) if matrix_coef else (self.int_dim[0],)
        self.weight_coef = nn.Parameter(torch.empty(coef_shape, dtype=dtype, device=device), requires_grad=True)
        self.register_buffer("weight", CreateRandumbTensor(self.weight_coef, self.seed[0], (out_features, in_features),
                                                           fused_bias=self.rt_bias))
        if bias:
            self.bias_coef = nn.Parameter(torch.empty(self.int_dim[1], dtype=dtype, device=device), requires_grad=True)
            self.register_buffer("bias", CreateRandumbTensor(self.bias_coef, self.seed[1], (out_features,), fused_bias=self.rt_bias))
        else:
            self.bias = None
        self.reset_parameters()

    def reset_parameters(self) -> None:
        self.init_zero_coef_uniform_bias()  # the reference's default (SillyLayers.py:218-221)

    def forward(self, input: torch.Tensor) -> torch.Tensor:
        if not self.fused:
            return F.linear(input, self.weight, self.bias)
        w = self.weight
        x2 = input.reshape(-1, self.in_features)
        if x2.dtype != w.dtype:
            x2 = x2.to(w.dtype)
        sb = w.scale_bias if w.fused_bias else None
        y = ops.linear(x2, self.weight_coef, self.in_features, self.out_features, self.in_features, 1, w.seed, sb, self.bias)
        return y.reshape(*input.shape[:-1], self.out_features)

    def extra_repr(self) -> str:
        return (f"in_features={self.in_features}, out_features={self.out_features}, int_dim={self.int_dim}, seeds={self.seed}, "
                f"bias={self.bias is not None}, matrix_coef={self.matrix_coef}, fused={self.fused}")

class SillyConv2d(SillyModuleMixin, nn.Conv2d):
    """``nn.Conv2d`` whose kernel (and bias) are vector-coef pseudorandom tensors.  Same constructor as the reference
    (SillyLayers.py:230-297): ``int_dim`` and ``seed`` are lists or generators yielding two values (weight, bias).

    The kernel is a 4-D pseudorandom tensor ``(out_channels, in_channels / groups, kh, kw)``: element ``a`` of its contiguous
    storage is ``sum_m noise(PRIME*a + m) * coef[m]``.  The convolution itself is the stock one: the tensor materialises for
    the duration of ``aten.convolution`` and the kernel's gradient reaches the coefficients through
    :class:`RandumbTensorConstructor`.  (The reference passes the 4-D size and strides into a kernel that takes two of each,
    SillyLayers.py:282-287 with RandumbTensor.py:375-380; here N-D shapes materialise through their storage extent.)
    """

    num_seeds = 2

    def __init__(self, in_channels: int, out_channels: int, int_dim: Union[list, GeneratorType], seed: Union[list, GeneratorType],
                 kernel_size, stride=1, padding=0, dilation=1, groups: int = 1, bias: bool = True, rt_bias: bool = False,
                 padding_mode: str = "zeros", device=None, dtype=None) -> None:
        self.int_dim = _take(int_dim, self.num_seeds)
        self.seed = _take(seed, self.num_seeds)
        self.rt_bias = rt_bias
        super().__init__(in_channels, out_channels, kernel_size, stride, padding, dilation, groups, bias, padding_mode,
                         device=device, dtype=dtype)

    def reset_parameters(self) -> None:
        # nn.Conv2d.__init__ has made dense parameters; keep their shapes, replace them (SillyLayers.py:280-294)
        w = self.weight
        self.weight_coef = nn.Parameter(torch.empty(self.int_dim[0], dtype=w.dtype, device=w.device), requires_grad=True)
        del self.weight
        self.register_buffer("weight", CreateRandumbTensor(self.weight_coef, self.seed[0], tuple(w.shape), fused_bias=self.rt_bias))
        if self.bias is not None:
            b = self.bias
            self.bias_coef = nn.Parameter(torch.empty(self.int_dim[1], dtype=b.dtype, device=b.device), requires_grad=True)
            del self.bias
            self.register_buffer("bias", CreateRandumbTensor(self.bias_coef, self.seed[1], tuple(b.shape), fused_bias=self.rt_bias))
        self.init_zero_coef_uniform_bias()

    def extra_repr(self) -> str:
        return f"{super().extra_repr()}, int_dim={self.int_dim}, seeds={self.seed}"


class SillyEmbedding(SillyModuleMixin, nn.Module):
    """Embedding whose table is a vector-coef pseudorandom tensor; only the requested rows are ever generated
    (SillyLayers.py:300-366).  ``padding_idx`` is not supported."""

    num_seeds = 1

    def __init__(self, num_embeddings: int, embedding_dim: int, int_dim: Union[list, GeneratorType], seed: Union[list, GeneratorType],
                 rt_bias: bool = False, padding_idx: Optional[int] = None, device="cuda", dtype=None) -> None:
        super().__init__()
        assert padding_idx is None, "padding_idx not supported"
        self.num_embeddings = num_embeddings
        self.embedding_dim = embedding_dim
        self.rt_bias = rt_bias
        self.padding_idx = None
        self.int_dim = _take(int_dim, self.num_seeds)
        self.seed = _take(seed, self.num_seeds)
        self.weight_coef = nn.Parameter(torch.empty(self.int_dim[0], dtype=dtype, device=device), requires_grad=True)
        self.register_buffer("weight", CreateRandumbTensor(self.weight_coef, self.seed[0], (num_embeddings, embedding_dim)))
        self.bias = None
        self.reset_parameters()

    def reset_parameters(self) -> None:
        if self.rt_bias:
            self.init_rt_scale_bias()
        init_kaiming_uniform(self.weight, None, seed=self.seed[0])

    def forward(self, input: torch.Tensor) -> torch.Tensor:
        return ops.embed_fwd(input, self.weight_coef, self.embedding_dim, self.weight.seed)

    def extra_repr(self) -> str:
        return f"{self.num_embeddings}, {self.embedding_dim}, int_dim={self.int_dim}, seeds={self.seed}"
