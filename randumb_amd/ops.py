"""``torch.library`` operators of the pseudorandom tensor, same names and argument meaning as the reference's
``rten::`` ops (src/rten_cpp/RandumbTensor.py:371-448, 1121-1157) and ``rten_cpp::`` ops
(src/rten_cpp/csrc/rten.cpp:36-39, src/rten_cpp/ops.py:9-13), implemented by the HIP kernels in
``librandumb_hip.so``.  CPU tensors raise ``NotImplementedError`` as they do in the reference.

Additive to the reference surface:
* ``materialize_fwd`` accepts a 2-D ``coefs`` (matrix-coef form) and declares ``scale_bias`` optional
  (the reference types it ``Tensor`` yet documents ``None`` as the default, RandumbTensor.py:993);
* ``materialize_bwd`` takes an optional ``coef_rows``;
* ``rten::linear_fwd`` / ``linear_bwd_dx`` / ``linear_bwd_dcoef``: the fused products that never write the
  weight (or its gradient) to memory.
"""
from __future__ import annotations

from typing import List, Optional

import torch
from torch import Tensor
from torch.library import custom_op

from . import hip

__all__ = [
    "materialize_fwd", "materialize_bwd", "scale_bias_bwd", "embed_fwd", "embed_bwd",
    "linear_fwd", "linear_bwd_dx", "linear_bwd_dcoef", "linear", "linear_project", "linear_project_fwd", "linear_fwd_projected",
    "linear_bwd_dcoef_projected", "linear_bwd_projected", "sq5_gen_2d", "sq5_gen_1d",
]


# ------------------------------------------------------------------------------------------------ rten::materialize_*
@custom_op("rten::materialize_fwd", mutates_args=())
def materialize_fwd(coefs: Tensor, size: List[int], strides: List[int], seed: int, scale_bias: Optional[Tensor],
                    fused_bias: bool, row_len: int = 0) -> Tensor:
    return hip.materialize_fwd(coefs, size, strides, seed, scale_bias, fused_bias, row_len if row_len > 0 else None)


@materialize_fwd.register_fake
def _(coefs, size, strides, seed, scale_bias, fused_bias, row_len=0):
    return coefs.new_empty(list(size), dtype=torch.float32)


@custom_op("rten::materialize_bwd", mutates_args=())
def materialize_bwd(dout: Tensor, dcoefs_size: int, seed: int, coef_rows: int = 0) -> Tensor:
    return hip.materialize_bwd(dout, dcoefs_size, seed, coef_rows)


@materialize_bwd.register_fake
def _(dout, dcoefs_size, seed, coef_rows=0):
    shape = [dcoefs_size] if coef_rows == 0 else [coef_rows, dcoefs_size]
    return dout.new_empty(shape, dtype=torch.float32)


@custom_op("rten::scale_bias_bwd", mutates_args=())
def scale_bias_bwd(dout: Tensor, seed: int) -> Tensor:
    return hip.scale_bias_bwd(dout, seed)


@scale_bias_bwd.register_fake
def _(dout, seed):
    return dout.new_empty([1], dtype=torch.float32)


def _to_base_layout(grad: Tensor, size, strides) -> Tensor:
    """Gradient of a strided view scattered back to the storage order the noise rows are numbered in."""
    size, strides = list(size), list(strides)
    contiguous = [1] * len(size)
    for i in range(len(size) - 2, -1, -1):
        contiguous[i] = contiguous[i + 1] * size[i + 1]
    if strides == contiguous or grad.numel() == 0:
        return grad.contiguous().flatten()
    extent = 1 + sum((s - 1) * st for s, st in zip(size, strides))
    base = grad.new_zeros(extent)
    base.as_strided(size, strides).copy_(grad)
    return base


def _mat_setup_context(ctx, inputs, output):
    coefs, size, strides, seed, scale_bias, fused_bias, row_len = inputs
    ctx.k = coefs.shape[-1]
    ctx.coef_rows = 0 if coefs.dim() == 1 else coefs.shape[0]
    ctx.coef_dtype = coefs.dtype
    ctx.size, ctx.strides, ctx.seed, ctx.fused_bias = list(size), list(strides), seed, fused_bias
    ctx.sb_dtype = None if scale_bias is None else scale_bias.dtype


def _mat_backward(ctx, grad):
    # only coefs and scale_bias are differentiable (RandumbTensor.py:423-428)
    g = _to_base_layout(grad, ctx.size, ctx.strides)
    dcoefs = materialize_bwd(g, ctx.k, ctx.seed, ctx.coef_rows).to(ctx.coef_dtype)
    dscale_bias = scale_bias_bwd(g, ctx.seed).to(ctx.sb_dtype) if ctx.fused_bias else None
    return dcoefs, None, None, None, dscale_bias, None, None


materialize_fwd.register_autograd(_mat_backward, setup_context=_mat_setup_context)


# ------------------------------------------------------------------------------------------------ rten::embed_*
@custom_op("rten::embed_fwd", mutates_args=())
def embed_fwd(idx: Tensor, coefs: Tensor, rowsize: int, seed: int) -> Tensor:
    return hip.embed_fwd(idx, coefs, rowsize, seed)


@embed_fwd.register_fake
def _(idx, coefs, rowsize, seed):
    return coefs.new_empty([*idx.shape, rowsize], dtype=torch.float32)


@custom_op("rten::embed_bwd", mutates_args=())
def embed_bwd(idx: Tensor, dout: Tensor, dcoefs_size: int, rowsize: int, seed: int) -> Tensor:
    return hip.embed_bwd(idx, dout.contiguous(), dcoefs_size, rowsize, seed)


@embed_bwd.register_fake
def _(idx, dout, dcoefs_size, rowsize, seed):
    return dout.new_empty([dcoefs_size], dtype=torch.float32)


def _embed_setup_context(ctx, inputs, output):
    idx, coefs, rowsize, seed = inputs
    ctx.save_for_backward(idx)
    ctx.dcoefs_size, ctx.rowsize, ctx.seed, ctx.coef_dtype = coefs.numel(), rowsize, seed, coefs.dtype


def _embed_backward(ctx, grad):
    (idx,) = ctx.saved_tensors
    return None, embed_bwd(idx, grad, ctx.dcoefs_size, ctx.rowsize, ctx.seed).to(ctx.coef_dtype), None, None


embed_fwd.register_autograd(_embed_backward, setup_context=_embed_setup_context)


# ------------------------------------------------------------------------------------------------ rten::linear_*
@custom_op("rten::linear_fwd", mutates_args=())
def linear_fwd(x: Tensor, coefs: Tensor, in_features: int, out_features: int, stride_o: int, stride_i: int, seed: int,
               scale_bias: Optional[Tensor], bias: Optional[Tensor]) -> Tensor:
    return hip.linear_fwd(x, coefs, in_features, out_features, stride_o, stride_i, seed, scale_bias, bias)


@linear_fwd.register_fake
def _(x, coefs, in_features, out_features, stride_o, stride_i, seed, scale_bias, bias):
    return x.new_empty([x.shape[0], out_features])


@custom_op("rten::linear_bwd_dx", mutates_args=())
def linear_bwd_dx(dy: Tensor, coefs: Tensor, in_features: int, out_features: int, stride_o: int, stride_i: int, seed: int,
                  scale_bias: Optional[Tensor]) -> Tensor:
    return hip.linear_bwd_dx(dy, coefs, in_features, out_features, stride_o, stride_i, seed, scale_bias)


@linear_bwd_dx.register_fake
def _(dy, coefs, in_features, out_features, stride_o, stride_i, seed, scale_bias):
    return dy.new_empty([dy.shape[0], in_features])


@custom_op("rten::linear_bwd_dcoef", mutates_args=())
def linear_bwd_dcoef(dy: Tensor, x: Tensor, dcoefs_size: int, coef_rows: int, in_features: int, out_features: int,
                     stride_o: int, stride_i: int, seed: int, want_scale_bias_grad: bool) -> List[Tensor]:
    dcoef, dsb = hip.linear_bwd_dcoef(dy, x, dcoefs_size, coef_rows, in_features, out_features, stride_o, stride_i, seed,
                                      want_scale_bias_grad)
    return [dcoef] if dsb is None else [dcoef, dsb]


@linear_bwd_dcoef.register_fake
def _(dy, x, dcoefs_size, coef_rows, in_features, out_features, stride_o, stride_i, seed, want_scale_bias_grad):
    shape = [dcoefs_size] if coef_rows == 0 else [coef_rows, dcoefs_size]
    out = [dy.new_empty(shape, dtype=torch.float32)]
    if want_scale_bias_grad:
        out.append(dy.new_empty([1], dtype=torch.float32))
    return out


def _lin_setup_context(ctx, inputs, output):
    x, coefs, in_features, out_features, stride_o, stride_i, seed, scale_bias, bias = inputs
    ctx.save_for_backward(x, coefs, scale_bias)
    ctx.meta = (in_features, out_features, stride_o, stride_i, seed)
    ctx.has_bias = bias is not None
    ctx.bias_dtype = None if bias is None else bias.dtype


def _lin_backward(ctx, dy):
    x, coefs, scale_bias = ctx.saved_tensors
    in_f, out_f, sO, sI, seed = ctx.meta
    dy = dy.contiguous()
    dx = dcoefs = dsb = dbias = None
    if ctx.needs_input_grad[0]:
        dx = linear_bwd_dx(dy, coefs, in_f, out_f, sO, sI, seed, scale_bias)
    want_sb = scale_bias is not None and ctx.needs_input_grad[7]
    if ctx.needs_input_grad[1] or want_sb:
        res = linear_bwd_dcoef(dy, x, coefs.shape[-1], 0 if coefs.dim() == 1 else coefs.shape[0], in_f, out_f, sO, sI, seed,
                               want_sb)
        dcoefs = res[0].to(coefs.dtype)
        if want_sb:
            dsb = res[1].to(scale_bias.dtype)
    if ctx.has_bias and ctx.needs_input_grad[8]:
        dbias = dy.sum(0).to(ctx.bias_dtype)
    return dx, dcoefs, None, None, None, None, None, dsb, dbias


linear_fwd.register_autograd(_lin_backward, setup_context=_lin_setup_context)


# ------------------------------------------------------------------------------------------------ projected form
@custom_op("rten::linear_project", mutates_args=())
def linear_project(x: Tensor, dcoefs_size: int, out_features: int, seed: int, coefs: Optional[Tensor]) -> Tensor:
    """Projection state of ``x`` (a byte tensor): ``z = x @ Noise.T`` (tokens, k), what the forward product and the coef
    gradient of a matrix-coef layer need of x, plus, when ``coefs`` is given, the transposed coefficients for the input
    gradient."""
    return hip.linear_project(x, dcoefs_size, out_features, seed, coefs)


@linear_project.register_fake
def _(x, dcoefs_size, out_features, seed, coefs):
    # the size is the library's business; a fake tensor only needs some 1-D byte shape
    nbytes = hip.linear_projection_bytes(x.shape[0], x.shape[1], out_features, dcoefs_size, x.dtype)
    return x.new_empty([x.shape[0], -(-nbytes // x.shape[0])], dtype=torch.uint8)


@custom_op("rten::linear_fwd_projected", mutates_args=())
def linear_fwd_projected(state: Tensor, coefs: Tensor, in_features: int, seed: int, bias: Optional[Tensor]) -> Tensor:
    """bf16 coefficients: the state of a bf16 layer; fp32 coefficients: that of an fp32 layer."""
    return hip.linear_fwd_projected(state, coefs, in_features, seed, bias, f32_state=coefs.dtype == torch.float32)


@linear_fwd_projected.register_fake
def _(state, coefs, in_features, seed, bias):
    return coefs.new_empty([state.shape[0], coefs.shape[0]])


@custom_op("rten::linear_project_fwd", mutates_args=())
def linear_project_fwd(x: Tensor, coefs: Tensor, seed: int, bias: Optional[Tensor]) -> List[Tensor]:
    """``[y, state]``: ``linear_project`` with the coefficients and ``linear_fwd_projected`` in one call (one kernel launch
    for k <= 256)."""
    y, state = hip.linear_project_fwd(x, coefs, seed, bias)
    return [y, state]


@linear_project_fwd.register_fake
def _(x, coefs, seed, bias):
    nbytes = hip.linear_projection_bytes(x.shape[0], x.shape[1], coefs.shape[0], coefs.shape[1], x.dtype)
    return [x.new_empty([x.shape[0], coefs.shape[0]]),
            x.new_empty([x.shape[0], -(-nbytes // x.shape[0])], dtype=torch.uint8)]


@custom_op("rten::linear_bwd_dcoef_projected", mutates_args=())
def linear_bwd_dcoef_projected(dy: Tensor, state: Tensor, dcoefs_size: int, in_features: int, seed: int) -> Tensor:
    return hip.linear_bwd_dcoef_projected(dy, state, dcoefs_size, in_features, seed)


@linear_bwd_dcoef_projected.register_fake
def _(dy, state, dcoefs_size, in_features, seed):
    return dy.new_empty([dy.shape[1], dcoefs_size], dtype=torch.float32)


@custom_op("rten::linear_bwd_projected", mutates_args=())
def linear_bwd_projected(dy: Tensor, state: Tensor, coefs: Tensor, in_features: int, seed: int) -> List[Tensor]:
    """``[dx, dcoef]`` of a matrix-coef bf16 layer from the projection state, in one call."""
    dx, dcoef = hip.linear_bwd_projected(dy, state, coefs, in_features, seed)
    return [dx, dcoef]


@linear_bwd_projected.register_fake
def _(dy, state, coefs, in_features, seed):
    return [dy.new_empty([dy.shape[0], in_features]), dy.new_empty([coefs.shape[0], coefs.shape[1]], dtype=torch.float32)]


def _tracing() -> bool:
    return torch.compiler.is_compiling()


def _dense(t: Optional[Tensor]) -> Optional[Tensor]:
    """A pseudorandom tensor (a random-backed bias) as the dense tensor the library reads; the operator wrappers get this from
    the tensor subclass's dispatch, the direct calls have to ask for it."""
    return t.get_materialized() if t is not None and hasattr(t, "get_materialized") else t


class _EagerLinear(torch.autograd.Function):
    """``rten::linear_fwd`` and its registered backward, without the operator wrappers: what ``linear`` runs eagerly."""

    @staticmethod
    def forward(ctx, x, coefs, in_features, out_features, stride_o, stride_i, seed, scale_bias, bias):
        ctx.save_for_backward(x, coefs, scale_bias)
        ctx.meta = (in_features, out_features, stride_o, stride_i, seed)
        ctx.bias_dtype = None if bias is None else bias.dtype
        return hip.linear_fwd(x, coefs, in_features, out_features, stride_o, stride_i, seed, scale_bias, _dense(bias))

    @staticmethod
    def backward(ctx, dy):
        x, coefs, scale_bias = ctx.saved_tensors
        in_f, out_f, sO, sI, seed = ctx.meta
        dy = dy.contiguous()
        dx = dcoefs = dsb = dbias = None
        want_sb = scale_bias is not None and ctx.needs_input_grad[7]
        if ctx.needs_input_grad[0] and want_sb and sO == in_f and sI == 1:
            # the random-bias product dy.R that dx needs anyway also gives the gradient of the bias's scale (reduced against x in
            # the same pass), so the coefficient gradient below comes from the factored kernels and dW is never formed
            both = hip.linear_bwd_dx_dscale(dy, x, coefs, in_f, out_f, seed, scale_bias)
            if both is not None:
                dx, dsb = both[0], both[1].to(scale_bias.dtype)
                want_sb = False
        if ctx.needs_input_grad[0] and dx is None:
            dx = hip.linear_bwd_dx(dy, coefs, in_f, out_f, sO, sI, seed, scale_bias)
        if ctx.needs_input_grad[1] or want_sb:
            dc, ds = hip.linear_bwd_dcoef(dy, x, coefs.shape[-1], 0 if coefs.dim() == 1 else coefs.shape[0], in_f, out_f, sO, sI, seed, want_sb)
            dcoefs = dc.to(coefs.dtype)
            if want_sb:
                dsb = ds.to(scale_bias.dtype)
        if ctx.bias_dtype is not None and ctx.needs_input_grad[8]:
            dbias = dy.sum(0).to(ctx.bias_dtype)
        return dx, dcoefs, None, None, None, None, None, dsb, dbias


class _ProjectedLinear(torch.autograd.Function):
    """``y = x @ W.T (+ bias)`` for a matrix-coef weight in bf16 or fp32.  The forward pass computes the projection state
    (``z = x @ Noise.T`` in the element orders its consumers read, and for bf16 the transposed coefficients) once and saves it
    for the backward pass, which then needs nothing else of ``x``; the reference's autograd saves ``x`` and materialises ``W``
    again (RandumbTensor.py:942-946, 979-990).  Per token the bf16 state holds 4 bytes per coefficient (k rounded up to 64)
    where x holds 2 per input feature, plus once per layer a copy of the coefficients; ``x`` itself usually stays alive too
    (its producer saved it), so ``linear`` takes this function only while the state is at most twice the size of x
    (``hip.linear_projection_preferred``).  With the fused random bias (``scale_bias``, bf16, eager only) the full-rank share
    ``s.R`` is added by kernels of its own in both directions and ``x`` is saved as well: the gradient of ``s`` is
    ``<dy @ R, x>``."""

    @staticmethod
    def forward(ctx, x, coefs, in_features, out_features, seed, bias, scale_bias=None):
        # eagerly: straight to the library (the operator wrappers of torch.library cost more host time than the layer's
        # kernels take); under torch.compile: through the registered operators, which it can trace
        y, state = linear_project_fwd(x, coefs, seed, bias) if _tracing() else hip.linear_project_fwd(x, coefs, seed, _dense(bias))
        if scale_bias is not None:
            hip.linear_rbias_fwd_(y, x, scale_bias, in_features, out_features, seed)
            ctx.save_for_backward(state, coefs, scale_bias, x)
        else:
            ctx.save_for_backward(state, coefs)
        ctx.meta = (in_features, out_features, seed)
        ctx.bias_dtype = None if bias is None else bias.dtype
        return y

    @staticmethod
    def backward(ctx, dy):
        state, coefs = ctx.saved_tensors[:2]
        scale_bias, x = ctx.saved_tensors[2:] if len(ctx.saved_tensors) == 4 else (None, None)
        in_f, out_f, seed = ctx.meta
        if dy.stride(-1) != 1 or dy.stride(0) < dy.shape[1] or dy.stride(0) % 8 or dy.data_ptr() % 16:
            dy = dy.contiguous()   # the kernels read rows with a leading dimension; anything else is copied
        dx = dcoefs = dbias = dsb = None
        direct = not _tracing()
        want_sb = scale_bias is not None and ctx.needs_input_grad[6]
        want_dx = ctx.needs_input_grad[0] or want_sb   # the gradient of the scale comes out of the random-bias share of dx
        if want_dx and ctx.needs_input_grad[1]:
            if direct:   # the sums leave the kernel in the coefficients' dtype: no cast afterwards
                dx, dcoefs = hip.linear_bwd_projected(dy, state, coefs, in_f, seed, dcoef_dtype=coefs.dtype)
            else:
                dx, dc = linear_bwd_projected(dy, state, coefs, in_f, seed)
                dcoefs = dc.to(coefs.dtype)
        elif want_dx:
            dx = (hip.linear_bwd_dx(dy, coefs, in_f, out_f, in_f, 1, seed, None) if direct
                  else linear_bwd_dx(dy, coefs, in_f, out_f, in_f, 1, seed, None))
        elif ctx.needs_input_grad[1]:
            if coefs.dtype == torch.float32:   # fp32 sums over token ranges need the backward call's workspace
                dcoefs = hip.linear_bwd_projected(dy, state, coefs, in_f, seed, want_dx=False)[1]
            else:
                dc = (hip.linear_bwd_dcoef_projected(dy, state, coefs.shape[1], in_f, seed) if direct
                      else linear_bwd_dcoef_projected(dy, state, coefs.shape[1], in_f, seed))
                dcoefs = dc.to(coefs.dtype)
        if scale_bias is not None and dx is not None:
            ds = hip.linear_rbias_bwd_(dx, dy, x, scale_bias, in_f, out_f, seed, want_scale_bias_grad=want_sb)
            if want_sb:
                dsb = ds.to(scale_bias.dtype)
        if not ctx.needs_input_grad[0]:
            dx = None
        if ctx.bias_dtype is not None and ctx.needs_input_grad[5]:
            dbias = dy.sum(0).to(ctx.bias_dtype)
        return dx, dcoefs, None, None, None, dbias, dsb


def linear(x: Tensor, coefs: Tensor, in_features: int, out_features: int, stride_o: int, stride_i: int, seed: int,
           scale_bias: Optional[Tensor], bias: Optional[Tensor]) -> Tensor:
    """``x @ W.T (+ bias)`` with autograd, choosing the projected form when the layer qualifies (matrix-coef; bf16 with sizes in
    multiples of 8, or fp32 beyond the few-token regime; the fused random bias in bf16 when run eagerly) and
    ``rten::linear_fwd`` otherwise.  Same arguments as ``rten::linear_fwd``."""
    rbias_ok = scale_bias is None or (x.dtype == torch.bfloat16 and scale_bias.numel() == 1 and not _tracing()
                                      and hip.linear_rbias_supported(in_features, out_features, x.dtype))
    if (rbias_ok and coefs.dim() == 2 and coefs.shape[0] == out_features and stride_o == in_features and stride_i == 1
            and x.is_cuda and x.dim() == 2 and x.dtype in (torch.bfloat16, torch.float32) and coefs.dtype == x.dtype
            and (bias is None or bias.dtype == x.dtype)
            and hip.linear_projection_preferred(x.shape[0], in_features, out_features, coefs.shape[1], x.dtype)):
        return _ProjectedLinear.apply(x, coefs, in_features, out_features, seed, bias, scale_bias)
    if x.is_cuda and not _tracing():
        return _EagerLinear.apply(x, coefs, in_features, out_features, stride_o, stride_i, seed, scale_bias, bias)
    return linear_fwd(x, coefs, in_features, out_features, stride_o, stride_i, seed, scale_bias, bias)


# ------------------------------------------------------------------------------------------------ rten_cpp::*
@custom_op("rten_cpp::sq5_gen_2d", mutates_args=())
def _sq5_gen_2d(M: int, N: int, seed: int) -> Tensor:
    return hip.sq5_fill_2d(M, N, seed)


@_sq5_gen_2d.register_fake
def _(M, N, seed):
    return torch.empty([M, N], dtype=torch.float32, device="cuda")


@custom_op("rten_cpp::materialize_fwd", mutates_args=())
def _cpp_materialize_fwd(coef: Tensor, seed: int, P: int, Q: int, stride_P: int, stride_Q: int) -> Tensor:
    assert coef.dim() == 1 and coef.is_contiguous()  # rten.cu:130-131
    return hip.materialize_fwd(coef, (P, Q), (stride_P, stride_Q), seed, None, False)


@_cpp_materialize_fwd.register_fake
def _(coef, seed, P, Q, stride_P, stride_Q):
    return coef.new_empty([P, Q], dtype=torch.float32)


def sq5_gen_2d(M: int, N: int, seed: int) -> Tensor:
    """Noise matrix ``(M, N)``; wrapper with the reference's name (src/rten_cpp/ops.py:9-10)."""
    return torch.ops.rten_cpp.sq5_gen_2d.default(M, N, seed)


def sq5_gen_1d(N: int, seed: int) -> Tensor:
    return hip.sq5_fill_1d(N, seed)
