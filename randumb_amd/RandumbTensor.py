"""``RandumbTensor``: a tensor whose values are ``Noise(seed) @ coef`` and are never stored.

Mirrors the reference's tensor subclass and its autograd constructor (src/rten_cpp/RandumbTensor.py:794-994):
a wrapper subclass that materialises itself for the duration of one aten op, keeps ``view / transpose / t /
permute / _to_copy`` lazy by only changing shape and strides, and back-propagates into the coefficient tensor
through ``RandumbTensorConstructor``.  Differences, all additive:

* ``coefs`` may be 2-D (matrix-coef form, one coef row per row of a ``(rows, row_len)`` tensor);
* ``aten.mm`` / ``aten.addmm`` against a dense CUDA matrix run the fused kernels, which regenerate the weight
  on chip instead of writing it to memory first (the reference materialises and calls a dense product,
  RandumbTensor.py:942-946).  ``RandumbTensor.FUSED_MM = False`` restores materialise-then-matmul.  Vector-coef tensors
  (the reference's form: k hashes per weight element) take materialise-then-matmul by default, because a fused product has
  to regenerate the whole weight for every block of 128 rows of the other matrix; ``RandumbTensor.FUSED_MM_VECTOR = True``
  gives them the fused kernels too (no transient weight in memory, at the price of that regeneration);
* ``_to_copy(dtype=...)`` yields a tensor that reports, and materialises to, the requested dtype.
"""
from __future__ import annotations

from collections.abc import Iterable
from typing import Optional, Union

import torch
from torch.autograd import Function
from torch.utils._pytree import tree_map

from . import ops

aten = torch.ops.aten


def _view_meta(func, shape, stride, args, kwargs):
    """Shape and stride the view op would produce, computed on a meta tensor (raises like the real op would,
    e.g. "view size is not compatible with input tensor's size and stride")."""
    fake = torch.empty_strided(tuple(shape), tuple(stride), device="meta")
    kwargs = {k: v for k, v in (kwargs or {}).items() if k not in ("device", "pin_memory", "non_blocking", "layout")}
    out = func(fake, *args, **kwargs)
    return out.shape, out.stride(), out.dtype


class RandumbTensor(torch.Tensor):
    """Structured tensor ``W_flat[a] = sum_m noise(PRIME*a + m) * coef[m]`` (vector-coef, ``coef`` is ``(k,)``) or
    ``W[o, i] = sum_m noise(PRIME*i + m) * coef[o, m]`` (matrix-coef, ``coef`` is ``(rows, k)``).

    Register ``_coef`` as a module parameter and the tensor itself as a buffer.  Always build it with
    :func:`CreateRandumbTensor` so gradients reach the coefficients.  The device is the coefficient's device and
    must be a GPU for any op that needs values; materialised values are fp32, then cast to ``dtype``.
    """

    FUSED_MM = True
    FUSED_MM_VECTOR = False

    @staticmethod
    def __new__(cls, data: torch.Tensor, seed: int, shape: Union[tuple, torch.Size], scale_bias: Optional[torch.Tensor],
                fused_bias: bool, strides: Optional[tuple] = None, dtype: Optional[torch.dtype] = None,
                row_len: Optional[int] = None):
        assert not data.requires_grad or not torch.is_grad_enabled()
        kwargs = {}
        if strides is not None:
            kwargs["strides"] = tuple(strides)
        return torch.Tensor._make_wrapper_subclass(cls, torch.Size(shape), device=data.device, dtype=dtype or data.dtype,
                                                   requires_grad=False, **kwargs)

    def __init__(self, data: torch.Tensor, seed: int, shape: Union[tuple, torch.Size], scale_bias: Optional[torch.Tensor],
                 fused_bias: bool, strides: Optional[tuple] = None, dtype: Optional[torch.dtype] = None,
                 row_len: Optional[int] = None):
        self.seed = seed
        self.scale_bias = scale_bias
        self.fused_bias = fused_bias
        self._coef = data
        size = self._coef.size()
        assert len(size) in (1, 2), f"Coefficient tensor must be 1D or 2D but received tensor of shape {size}"
        self.int_dim = size[-1]
        self.coef_rows = 0 if len(size) == 1 else size[0]
        if self.coef_rows:
            if row_len is None:
                assert len(shape) == 2 and shape[0] == self.coef_rows, \
                    f"matrix-coef of {self.coef_rows} rows needs a ({self.coef_rows}, row_len) shape, got {tuple(shape)}"
                row_len = shape[1]
            self.row_len = int(row_len)
        else:
            self.row_len = 0
        self._tensor: Optional[torch.Tensor] = None
        numel = 1
        for s in shape:
            numel *= s
        # shape of the noise matrix that is never stored
        self.noise_matrix_shape = torch.Size((self.row_len if self.coef_rows else numel, self.int_dim))

    def __repr__(self):
        with torch._C._DisableTorchDispatch():
            return (f"RandumbTensor(seed={self.seed}, int_dim={self.int_dim}, shape={self.shape}, stride={self.stride()}, "
                    f"noise_matrix_shape={self.noise_matrix_shape}, dtype={self.dtype}, device='{self.device}')")

    # -------------------------------------------------------------------------------------------- helpers
    def get_materialized(self) -> torch.Tensor:
        self.materialize()
        ref = self._tensor
        self.dematerialize()
        return ref

    def get_noise_matrix(self) -> torch.Tensor:
        return ops.sq5_gen_2d(self.noise_matrix_shape[0], self.noise_matrix_shape[1], self.seed)

    def print_memory(self):
        noise_mem = self.element_size() * self.noise_matrix_shape.numel() / 2**20
        coeff_mem = self._coef.element_size() * self._coef.numel() / 2**20
        out_mem = self.element_size() * self.shape.numel() / 2**20
        total_mem = noise_mem + coeff_mem + out_mem
        print(f"unmaterialized noise matrix: {noise_mem}MiB\ncoefficient matrix: {coeff_mem}MiB\noutput matrix: {out_mem}MiB")
        print(f"% 'saved' memory: {noise_mem / total_mem * 100}%")

    @torch.compiler.disable(recursive=False)
    def materialize(self):
        with torch.no_grad():
            size, stride = list(self.size()), list(self.stride())
            if len(size) == 0:
                size, stride = [1], [1]
            if len(size) > 2:
                # N-D views: materialise the flat storage extent and restride it
                extent = 1 + sum((s - 1) * st for s, st in zip(size, stride))
                flat = ops.materialize_fwd(self._coef.detach(), [extent], [1], self.seed, self._sb(), self.fused_bias, self.row_len)
                self._tensor = flat.as_strided(size, stride).contiguous().to(self.dtype)
            else:
                out = ops.materialize_fwd(self._coef.detach(), size, stride, self.seed, self._sb(), self.fused_bias, self.row_len)
                self._tensor = out.reshape(self.size()).to(self.dtype)

    def dematerialize(self):
        self._tensor = None

    def _sb(self):
        return None if self.scale_bias is None else self.scale_bias.detach()

    __torch_function__ = torch._C._disabled_torch_function_impl
    OVERRIDE_VIEW_OPS = [aten.view.default, aten.transpose.int, aten._to_copy.default, aten.t.default, aten.permute.default,
                         aten._unsafe_view.default, aten.detach.default, aten.alias.default]

    # -------------------------------------------------------------------------------------------- fused products
    def _fused_ok(self, other) -> bool:
        return (type(self).FUSED_MM and (self.coef_rows or type(self).FUSED_MM_VECTOR) and self.dim() == 2 and isinstance(other, torch.Tensor)
                and not isinstance(other, RandumbTensor) and other.is_cuda and other.dim() == 2
                and other.dtype in (torch.float32, torch.bfloat16) and other.dtype == self.dtype)

    def _rmm(self, mat1: torch.Tensor, bias: Optional[torch.Tensor] = None) -> Optional[torch.Tensor]:
        """``mat1 @ self`` (+ bias) on the fused kernels, or None when this layout has no fused kernel."""
        P, Q = self.shape
        sP, sQ = self.stride()
        sb = self._sb() if self.fused_bias else None
        coef = self._coef.detach()
        if not self.coef_rows:
            return ops.linear_fwd(mat1, coef, P, Q, sQ, sP, self.seed, sb, bias)
        if (P, Q, sP, sQ) == (self.row_len, self.coef_rows, 1, self.row_len):  # transposed base: x @ W.T
            return ops.linear_fwd(mat1, coef, P, Q, sQ, sP, self.seed, sb, bias)
        if (P, Q, sP, sQ) == (self.coef_rows, self.row_len, self.row_len, 1) and bias is None:  # base: dy @ W
            return ops.linear_bwd_dx(mat1, coef, Q, P, sP, sQ, self.seed, sb)
        return None

    @classmethod
    def __torch_dispatch__(cls, func, types, args=(), kwargs=None):
        kwargs = kwargs or {}
        if func in cls.OVERRIDE_VIEW_OPS:
            inst: RandumbTensor = args[0]
            with torch.no_grad():
                shape, stride, dtype = _view_meta(func, inst.shape, inst.stride(), args[1:], kwargs)
                if func is not aten._to_copy.default or kwargs.get("dtype") is None:
                    dtype = inst.dtype
                return RandumbTensor(inst._coef, inst.seed, shape, inst.scale_bias, inst.fused_bias, stride, dtype, inst.row_len or None)

        if func is aten.mm.default and not kwargs:
            a, b = args
            if isinstance(b, RandumbTensor) and b._fused_ok(a):
                out = b._rmm(a)
                if out is not None:
                    return out
            elif isinstance(a, RandumbTensor) and a._fused_ok(b):  # self @ mat2 = (mat2.T @ self.T).T
                out = a.t()._rmm(b.t().contiguous())
                if out is not None:
                    return out.t()
        elif func is aten.addmm.default and kwargs.get("beta", 1) == 1 and kwargs.get("alpha", 1) == 1:
            bias, a, b = args
            if isinstance(b, RandumbTensor) and b._fused_ok(a):
                dense_bias = bias.get_materialized() if isinstance(bias, RandumbTensor) else bias
                if dense_bias.dim() == 1 and dense_bias.shape[0] == b.shape[1]:
                    out = b._rmm(a, dense_bias)
                    if out is not None:
                        return out

        materialized = []

        def _materialize(e):
            if isinstance(e, RandumbTensor):
                e.materialize()
                materialized.append(e)
                return e._tensor
            return e

        ret = func(*tree_map(_materialize, args), **tree_map(_materialize, kwargs))
        for t in materialized:
            t.dematerialize()
        return ret


class RandumbTensorConstructor(Function):
    """Differentiable constructor: forward wraps the coefficients, backward maps the tensor's gradient to the
    coefficients with ``materialize_bwd`` (and ``scale_bias_bwd``).  Reference: RandumbTensor.py:959-990."""

    @staticmethod
    def forward(ctx, coefs: torch.Tensor, seed: int, shape: Iterable, scale_bias: Optional[torch.Tensor], fused_bias: bool) -> RandumbTensor:
        if not isinstance(coefs, torch.Tensor):
            raise AssertionError(f"Expected coefs to be of type torch.Tensor, found {type(coefs)} instead.")
        assert coefs.dim() in (1, 2), f"Coefficient tensor must be 1D or 2D but received tensor of shape {coefs.size()}"
        out = RandumbTensor(coefs, seed, tuple(shape), scale_bias, fused_bias)
        ctx.dcoefs_size = coefs.shape[-1]
        ctx.coef_rows = 0 if coefs.dim() == 1 else coefs.shape[0]
        ctx.seed = seed
        ctx.dtype = out.dtype
        ctx.fused_bias = fused_bias
        ctx.sb_dtype = None if scale_bias is None else scale_bias.dtype
        return out

    @staticmethod
    def backward(ctx, grad):
        grad = grad.contiguous().flatten()
        dcoefs = ops.materialize_bwd(grad, ctx.dcoefs_size, ctx.seed, ctx.coef_rows).to(ctx.dtype)
        dscale_bias = None
        if ctx.fused_bias:
            dscale_bias = ops.scale_bias_bwd(grad, ctx.seed).to(ctx.sb_dtype)
        return dcoefs, None, None, dscale_bias, None


def CreateRandumbTensor(coefs: torch.Tensor, seed: int, shape: Iterable, scale_bias: Optional[torch.Tensor] = None,
                        fused_bias: bool = False) -> RandumbTensor:
    """Use this, not the class, to build a ``RandumbTensor`` (reference: RandumbTensor.py:993-994)."""
    return RandumbTensorConstructor.apply(coefs, seed, shape, scale_bias, fused_bias)


def rt_mm(mat1: torch.Tensor, coefs: torch.Tensor, size, strides, seed: int, scale_bias: Optional[torch.Tensor],
          fused_bias: bool) -> torch.Tensor:
    """``mat1 (L, P) @ tensor (P, Q)`` without writing the tensor to memory; same signature as the reference's
    experimental ``rt_mm`` (RandumbTensor.py:634-645).  Returns ``(L, Q)`` in ``mat1``'s dtype."""
    P, Q = size
    assert mat1.size(1) == P, f"mm shape mismatch, received mat1 shape {mat1.size()} and rt shape {size}"
    assert not (fused_bias and scale_bias is None), "scale_bias not initialized but fused_bias is True"
    return ops.linear_fwd(mat1, coefs, P, Q, strides[1], strides[0], seed, scale_bias if fused_bias else None, None)
