"""Tensor-level wrappers over the C ABI: allocate outputs with torch, pass raw device pointers and the current
HIP stream to ``librandumb_hip.so``.  No arithmetic happens in Python and there is no CPU path: a CPU tensor
raises ``NotImplementedError`` exactly as the reference's CPU registrations do
(src/rten_cpp/RandumbTensor.py:438-448, 1151-1157)."""
from __future__ import annotations

import ctypes
import os
from typing import Optional, Sequence

import torch

from . import _lib
from ._lib import (LinearDesc, RDB_ALGO_AUTO, RDB_BF16, RDB_F32, RDB_OP_LINEAR_BWD_DCOEF, RDB_OP_LINEAR_BWD_DX,
                   RDB_OP_LINEAR_BWD_PROJECTED, RDB_OP_LINEAR_FWD)

_DT = {torch.float32: RDB_F32, torch.bfloat16: RDB_BF16}


def _need_gpu(name: str, *tensors) -> None:
    for t in tensors:
        if t is not None and not t.is_cuda:
            raise NotImplementedError(f"Unsupported CPU implementation of {name} called.")


def _native(t: Optional[torch.Tensor]) -> Optional[torch.Tensor]:
    """Contiguous tensor of a dtype the library reads directly (fp32 / bf16); other floats go through fp32."""
    if t is None:
        return None
    if t.dtype not in _DT:
        t = t.to(torch.float32)
    return t.contiguous()


def _p(t: Optional[torch.Tensor]):
    return None if t is None else ctypes.c_void_p(t.data_ptr())


def _stream(device) -> ctypes.c_void_p:
    idx = device.index
    return ctypes.c_void_p(torch._C._cuda_getCurrentRawStream(torch.cuda.current_device() if idx is None else idx))


class _NoSwitch:
    def __enter__(self):
        return None

    def __exit__(self, *exc):
        return False


_NO_SWITCH = _NoSwitch()


def _on(device):
    """Context in which ``device`` is the current device; no work when it already is (the usual case)."""
    idx = device.index
    return _NO_SWITCH if idx is None or idx == torch.cuda.current_device() else torch.cuda.device(idx)


def _workspace(nbytes: int, device) -> Optional[torch.Tensor]:
    # torch's caching allocator is the reusable pool: a block freed by the previous call on this stream comes back without
    # a device allocation, and blocks are never handed to another stream while work on them is pending
    return torch.empty(nbytes, dtype=torch.uint8, device=device) if nbytes > 0 else None


def _seed(seed: int) -> int:
    seed = int(seed)
    if not 0 <= seed < 2**32:
        raise ValueError(f"seed must fit in 32 unsigned bits, got {seed}")
    return seed


# ------------------------------------------------------------------------------------------------ waits that gave up
class SyncWatch:
    """Host side of the one-launch kernels' bounded waits.  A block that gives up waiting for blocks of its own launch fills
    its share of the output with NaN and adds one to a counter on the device; this object looks at that counter without ever
    making the hot loop wait: every ``every`` calls of an entry point that may run such a kernel it enqueues a 4-byte copy of
    the counter into pinned host memory behind the work already on the stream, and looks at the copy once the stream has got
    there.  A changed counter switches the library to separate launches (``rdb_set_one_launch(0)``) and raises."""

    def __init__(self, lib=None, host_word=None, event_factory=None, every: int = 64):
        self._lib = lib
        self._host = host_word
        self._event_factory = event_factory
        self.every = every
        self.calls = 0
        self.seen = 0
        self.pending = None

    def _library(self):
        return self._lib if self._lib is not None else _lib.load()

    def _host_word(self):
        if self._host is None:
            self._host = torch.zeros(1, dtype=torch.int32, pin_memory=True)
        return self._host

    def _enqueue(self, stream) -> None:
        L = self._library()
        _lib.check(L.rdb_sync_giveups_async(ctypes.c_void_p(self._host_word().data_ptr()), stream), "rdb_sync_giveups_async")
        ev = self._event_factory() if self._event_factory is not None else torch.cuda.Event()
        ev.record()
        self.pending = ev

    def _judge(self) -> None:
        self.pending = None
        count = int(self._host_word()[0]) & 0xFFFFFFFF
        if count != self.seen:
            new, self.seen = (count - self.seen) & 0xFFFFFFFF, count
            self._library().rdb_set_one_launch(0)
            raise _lib.RandumbHipError(
                f"{new} block(s) of a one-launch kernel gave up waiting for blocks of their own launch: the outputs they stood "
                "for were filled with NaN, and projection states and recorded graphs of those launches must not be used again. "
                "The library now runs producers and consumers as separate launches (rdb_set_one_launch(0)).")

    def tick(self, stream) -> None:
        """Called by the entry points that may run a one-launch kernel; never waits for the device."""
        self.calls += 1
        if self.pending is not None and self.pending.query():
            self._judge()
        if self.pending is None and self.calls % self.every == 0:
            self._enqueue(stream)

    def check(self, stream) -> None:
        """Waits for the work on ``stream`` and raises if any block gave up since the last look."""
        if self.pending is None:
            self._enqueue(stream)
        self.pending.synchronize()
        self._judge()


_watches: dict = {}


def _watch(device) -> SyncWatch:
    key = torch.device(device).index if torch.device(device).index is not None else torch.cuda.current_device()
    w = _watches.get(key)
    if w is None:
        w = _watches[key] = SyncWatch()
    return w


def sync_check(device="cuda") -> None:
    """Waits for the current stream of ``device`` and raises ``RandumbHipError`` if a block of a one-launch kernel has given
    up its bounded wait since the last look (a training loop may call this once per optimizer step; the entry points look by
    themselves, without waiting, every 64 calls)."""
    dev = torch.device(device)
    with torch.cuda.device(dev):
        _watch(dev).check(_stream(dev))


def set_one_launch(mode: int) -> int:
    """Process-wide: 0 = producers and consumers of the factored forward (and of the fp32 small-k products) always as
    separate launches, 1 = in one launch where that applies (default).  Same results bit for bit.  Returns the previous mode."""
    return int(_lib.load().rdb_set_one_launch(int(mode)))


def selftest_sync_giveup(y: torch.Tensor, scratch: torch.Tensor, coef: torch.Tensor, in_f: int, seed: int, polls: int = 64) -> None:
    """Test hook: runs only the consumer blocks of the one-launch forward of the layer ``coef`` (out_f, k) on ``scratch`` with
    a tag nobody publishes; every block gives up after ``polls`` polls, ``y`` becomes NaN and the give-up counter grows."""
    _need_gpu("selftest_sync_giveup", y, scratch, coef)
    d = _desc(y.shape[0], in_f, coef.shape[0], coef, in_f, 1, seed, y.dtype, RDB_ALGO_AUTO)
    with _on(y.device):
        rc = _lib.load().rdb_selftest_sync_giveup(_p(y), y.stride(0), _p(scratch), scratch.numel() * scratch.element_size(), _p(coef),
                                                  ctypes.byref(d), int(polls), _stream(y.device))
    _lib.check(rc, "rdb_selftest_sync_giveup")


# ------------------------------------------------------------------------------------------------ probes
def sq5_fill_2d(N: int, M: int, seed: int, device="cuda") -> torch.Tensor:
    """Noise matrix ``(N, M)``, ``out[n, m] = noise(PRIME*n + m)``  (RandumbTensor.py:101-105)."""
    out = torch.empty((N, M), dtype=torch.float32, device=device)
    _need_gpu("sq5_fill_2d", out)
    with _on(out.device):
        _lib.check(_lib.load().rdb_sq5_fill_2d(_p(out), N, M, _seed(seed), _stream(out.device)), "rdb_sq5_fill_2d")
    return out


def sq5_fill_1d(N: int, seed: int, device="cuda") -> torch.Tensor:
    """1-D noise ``out[n] = noise(n)``  (RandumbTensor.py:122-126)."""
    out = torch.empty((N,), dtype=torch.float32, device=device)
    _need_gpu("sq5_fill_1d", out)
    with _on(out.device):
        _lib.check(_lib.load().rdb_sq5_fill_1d(_p(out), N, _seed(seed), _stream(out.device)), "rdb_sq5_fill_1d")
    return out


# ------------------------------------------------------------------------------------------------ materialise
def materialize_fwd(coefs: torch.Tensor, size: Sequence[int], strides: Sequence[int], seed: int,
                    scale_bias: Optional[torch.Tensor], fused_bias: bool, row_len: Optional[int] = None) -> torch.Tensor:
    """fp32 contiguous tensor of shape ``size``; the view's ``strides`` address the noise rows
    (RandumbTensor.py:371-381).  ``coefs.dim() == 2`` selects the matrix-coef form, whose base tensor is
    ``(coefs.shape[0], row_len)`` contiguous (``row_len`` defaults to ``numel / coefs.shape[0]``)."""
    assert not (fused_bias and scale_bias is None), "scale_bias not initialized but fused_bias is True"
    _need_gpu("materialize_fwd", coefs)
    size, strides = [int(s) for s in size], [int(s) for s in strides]
    output = torch.empty(size, dtype=torch.float32, device=coefs.device)
    if len(size) == 1:  # RandumbTensor.py:375-377
        size, strides = [1, size[0]], [0, strides[0]]
    if len(size) != 2:
        raise ValueError(f"materialize_fwd supports 1-D and 2-D shapes, got {size}")
    c = _native(coefs)
    sb = _native(scale_bias).to(c.dtype) if fused_bias else None
    if c.dim() == 1:
        rows, k, row_len = 0, c.shape[0], 0
    elif c.dim() == 2:
        rows, k = c.shape
        numel = size[0] * size[1]
        if row_len is None:
            if rows == 0 or numel % rows:
                raise ValueError(f"matrix-coef with {rows} rows cannot back a tensor of {numel} elements")
            row_len = numel // rows
    else:
        raise ValueError("coefs must be 1-D or 2-D")
    with _on(c.device):
        rc = _lib.load().rdb_materialize_fwd(_p(output), _p(c), _DT[c.dtype], rows, k, row_len, size[0], size[1],
                                             strides[0], strides[1], _seed(seed), _p(sb), _stream(c.device))
    _lib.check(rc, "rdb_materialize_fwd")
    return output


def materialize_bwd(dout: torch.Tensor, dcoefs_size: int, seed: int, coef_rows: int = 0) -> torch.Tensor:
    """``Noise.T @ dout`` in fp32: ``(dcoefs_size,)`` or, matrix-coef, ``(coef_rows, dcoefs_size)``
    (RandumbTensor.py:383-390)."""
    assert dout.is_contiguous(), "dout is not contiguous, backwards pass might give incorrect results."
    _need_gpu("materialize_bwd", dout)
    d = _native(dout)
    k, Nw = int(dcoefs_size), d.numel()
    shape = (k,) if coef_rows == 0 else (coef_rows, k)
    row_len = 0 if coef_rows == 0 else Nw // max(coef_rows, 1)
    dcoefs = torch.empty(shape, dtype=torch.float32, device=d.device)
    L = _lib.load()
    with _on(d.device):
        ws_bytes = L.rdb_materialize_bwd_workspace_bytes(coef_rows, k, row_len, Nw)
        ws = _workspace(ws_bytes, d.device)
        rc = L.rdb_materialize_bwd(_p(dcoefs), _p(d), _DT[d.dtype], coef_rows, k, row_len, Nw, _seed(seed), _p(ws), ws_bytes,
                                   _stream(d.device))
    _lib.check(rc, "rdb_materialize_bwd")
    return dcoefs


def scale_bias_bwd(dout: torch.Tensor, seed: int) -> torch.Tensor:
    """``sum(dout * noise_1d)`` as an fp32 ``(1,)`` tensor (RandumbTensor.py:414-420)."""
    assert dout.is_contiguous(), "dout is not contiguous, backwards pass might give incorrect results."
    _need_gpu("scale_bias_bwd", dout)
    d = _native(dout)
    ds = torch.empty((1,), dtype=torch.float32, device=d.device)
    L = _lib.load()
    with _on(d.device):
        ws_bytes = L.rdb_scale_bias_bwd_workspace_bytes(d.numel())
        ws = _workspace(ws_bytes, d.device)
        rc = L.rdb_scale_bias_bwd(_p(ds), _p(d), _DT[d.dtype], d.numel(), _seed(seed), _p(ws), ws_bytes, _stream(d.device))
    _lib.check(rc, "rdb_scale_bias_bwd")
    return ds


# ------------------------------------------------------------------------------------------------ embedding
def embed_fwd(idx: torch.Tensor, coefs: torch.Tensor, rowsize: int, seed: int) -> torch.Tensor:
    """Rows ``idx`` of a ``(*, rowsize)`` vector-coef tensor, fp32 ``(*idx.shape, rowsize)`` (RandumbTensor.py:1121-1126)."""
    _need_gpu("embed_fwd", idx, coefs)
    c = _native(coefs)
    ix = idx.to(torch.int64).contiguous()
    out = torch.empty((*idx.shape, rowsize), dtype=torch.float32, device=c.device)
    with _on(c.device):
        rc = _lib.load().rdb_embed_fwd(_p(out), _p(ix), ix.numel(), _p(c), _DT[c.dtype], c.numel(), int(rowsize), _seed(seed),
                                       _stream(c.device))
    _lib.check(rc, "rdb_embed_fwd")
    return out


def embed_bwd(idx: torch.Tensor, dout: torch.Tensor, dcoefs_size: int, rowsize: int, seed: int) -> torch.Tensor:
    """Coefficient gradient of :func:`embed_fwd`, fp32 ``(dcoefs_size,)`` (RandumbTensor.py:1128-1134)."""
    _need_gpu("embed_bwd", idx, dout)
    d = _native(dout)
    ix = idx.to(torch.int64).contiguous()
    k = int(dcoefs_size)
    dcoefs = torch.empty((k,), dtype=torch.float32, device=d.device)
    L = _lib.load()
    with _on(d.device):
        ws_bytes = L.rdb_embed_bwd_workspace_bytes(ix.numel(), int(rowsize), k)
        ws = _workspace(ws_bytes, d.device)
        rc = L.rdb_embed_bwd(_p(dcoefs), _p(ix), ix.numel(), _p(d), _DT[d.dtype], k, int(rowsize), _seed(seed), _p(ws), ws_bytes,
                             _stream(d.device))
    _lib.check(rc, "rdb_embed_bwd")
    return dcoefs


# ------------------------------------------------------------------------------------------------ fused linear
def _desc(tokens, in_f, out_f, coef, sO, sI, seed, act_dtype, algo) -> LinearDesc:
    d = LinearDesc()
    d.tokens, d.in_f, d.out_f = int(tokens), int(in_f), int(out_f)
    d.k = int(coef.shape[-1])
    d.coef_rows = 0 if coef.dim() == 1 else int(coef.shape[0])
    d.sO, d.sI = int(sO), int(sI)
    d.seed = _seed(seed)
    d.act_dtype = _DT[act_dtype]
    d.coef_dtype = _DT[coef.dtype]
    d.algo = int(algo)
    return d


def _act(t: torch.Tensor) -> torch.Tensor:
    """2-D activation with unit inner stride in a dtype the kernels compute in."""
    if t.dtype not in _DT:
        t = t.to(torch.float32)
    if t.dim() != 2:
        raise ValueError("activations must be 2-D (tokens, features)")
    return t if t.stride(1) == 1 and t.stride(0) >= t.shape[1] else t.contiguous()


def linear_fwd(x: torch.Tensor, coef: torch.Tensor, in_f: int, out_f: int, sO: int, sI: int, seed: int,
               scale_bias: Optional[torch.Tensor] = None, bias: Optional[torch.Tensor] = None,
               algo: int = RDB_ALGO_AUTO) -> torch.Tensor:
    """``y = x @ W.T (+ bias)`` with the ``(out_f, in_f)`` pseudorandom weight regenerated on chip."""
    _need_gpu("linear_fwd", x, coef)
    x = _act(x)
    c = _native(coef)
    sb = None if scale_bias is None else _native(scale_bias).to(c.dtype)
    b = None if bias is None else bias.to(x.dtype).contiguous()
    y = torch.empty((x.shape[0], out_f), dtype=x.dtype, device=x.device)
    d = _desc(x.shape[0], in_f, out_f, c, sO, sI, seed, x.dtype, algo)
    L = _lib.load()
    with _on(x.device):
        ws_bytes = L.rdb_linear_workspace_bytes(RDB_OP_LINEAR_FWD, ctypes.byref(d))
        ws = _workspace(ws_bytes, x.device)
        st = _stream(x.device)
        rc = L.rdb_linear_fwd(_p(y), y.stride(0), _p(x), x.stride(0), _p(c), _p(sb), _p(b), ctypes.byref(d), _p(ws), ws_bytes, st)
        _lib.check(rc, "rdb_linear_fwd")
        _watch(x.device).tick(st)
    return y


def linear_bwd_dx(dy: torch.Tensor, coef: torch.Tensor, in_f: int, out_f: int, sO: int, sI: int, seed: int,
                  scale_bias: Optional[torch.Tensor] = None, algo: int = RDB_ALGO_AUTO) -> torch.Tensor:
    """``dx = dy @ W``."""
    _need_gpu("linear_bwd_dx", dy, coef)
    dy = _act(dy)
    c = _native(coef)
    sb = None if scale_bias is None else _native(scale_bias).to(c.dtype)
    dx = torch.empty((dy.shape[0], in_f), dtype=dy.dtype, device=dy.device)
    d = _desc(dy.shape[0], in_f, out_f, c, sO, sI, seed, dy.dtype, algo)
    L = _lib.load()
    with _on(dy.device):
        ws_bytes = L.rdb_linear_workspace_bytes(RDB_OP_LINEAR_BWD_DX, ctypes.byref(d))
        ws = _workspace(ws_bytes, dy.device)
        st = _stream(dy.device)
        rc = L.rdb_linear_bwd_dx(_p(dx), dx.stride(0), _p(dy), dy.stride(0), _p(c), _p(sb), ctypes.byref(d), _p(ws), ws_bytes, st)
        _lib.check(rc, "rdb_linear_bwd_dx")
        _watch(dy.device).tick(st)
    return dx


def linear_bwd_dx_dscale(dy: torch.Tensor, x: torch.Tensor, coef: torch.Tensor, in_f: int, out_f: int, seed: int, scale_bias: torch.Tensor):
    """``(dx, d_scale_bias)`` of a matrix-coef bf16 layer with the fused random bias: ``dx = dy @ W`` and the gradient of the
    bias's scale, ``<dy @ R, x>`` (fp32, ``(1,)``), from one pass over the random-bias product.  ``None`` when the library has
    no such kernel for the request (other dtypes or forms: the caller takes ``linear_bwd_dx`` and ``linear_bwd_dcoef``)."""
    _need_gpu("linear_bwd_dx_dscale", dy, x, coef, scale_bias)
    if dy.dtype != torch.bfloat16 or coef.dtype != torch.bfloat16 or coef.dim() != 2:
        return None
    dy, x = _act(dy), _act(x)
    if x.dtype != dy.dtype:
        x = x.to(dy.dtype)
    c = _native(coef)
    sb = _native(scale_bias).to(c.dtype)
    d = _desc(dy.shape[0], in_f, out_f, c, in_f, 1, seed, dy.dtype, RDB_ALGO_AUTO)
    L = _lib.load()
    ws_bytes = int(L.rdb_linear_workspace_bytes(_lib.RDB_OP_LINEAR_BWD_DX_DSCALE, ctypes.byref(d)))
    if ws_bytes <= 0:
        return None
    dx = torch.empty((dy.shape[0], in_f), dtype=dy.dtype, device=dy.device)
    ds = torch.empty((1,), dtype=torch.float32, device=dy.device)
    with _on(dy.device):
        ws = _workspace(ws_bytes, dy.device)
        rc = L.rdb_linear_bwd_dx_dscale(_p(dx), dx.stride(0), _p(ds), _p(dy), dy.stride(0), _p(x), x.stride(0), _p(c), _p(sb), ctypes.byref(d),
                                        _p(ws), ws_bytes, _stream(dy.device))
    if rc == -5:   # RDB_E_UNSUPPORTED: nothing was launched
        return None
    _lib.check(rc, "rdb_linear_bwd_dx_dscale")
    return dx, ds


def _rbias_desc(tokens: int, in_f: int, out_f: int, seed: int) -> LinearDesc:
    d = LinearDesc()
    d.tokens, d.in_f, d.out_f, d.k, d.coef_rows, d.sO, d.sI, d.seed = int(tokens), int(in_f), int(out_f), 8, int(out_f), int(in_f), 1, _seed(seed)
    d.act_dtype, d.coef_dtype, d.algo = _lib.RDB_BF16, _lib.RDB_BF16, RDB_ALGO_AUTO
    return d


def linear_rbias_supported(in_f: int, out_f: int, dtype) -> bool:
    """Whether the random-bias share has kernels of its own for the layer (bf16, sizes in multiples of 8)."""
    return dtype == torch.bfloat16 and in_f % 8 == 0 and out_f % 8 == 0


def linear_rbias_fwd_(y: torch.Tensor, x: torch.Tensor, scale_bias: torch.Tensor, in_f: int, out_f: int, seed: int) -> torch.Tensor:
    """In place: ``y += scale_bias * x @ R.T`` with ``R[o, i] = noise1d(o * in_f + i)``, the fused random bias of a weight
    ``W = C.N + s.R`` (src/rten_cpp/RandumbTensor.py:286-289), on top of a ``y`` that holds the low-rank share.  bf16."""
    _need_gpu("linear_rbias_fwd_", y, x, scale_bias)
    x = _act(x)
    sb = _native(scale_bias).to(torch.bfloat16)
    d = _rbias_desc(x.shape[0], in_f, out_f, seed)
    with _on(x.device):
        _lib.check(_lib.load().rdb_linear_rbias_fwd(_p(y), y.stride(0), _p(x), x.stride(0), _p(sb), ctypes.byref(d), _stream(x.device)),
                   "rdb_linear_rbias_fwd")
    return y


def linear_rbias_bwd_(dx: torch.Tensor, dy: torch.Tensor, x: Optional[torch.Tensor], scale_bias: torch.Tensor, in_f: int, out_f: int,
                      seed: int, want_scale_bias_grad: bool = False) -> Optional[torch.Tensor]:
    """In place: ``dx += scale_bias * dy @ R``; returns the gradient of the scale, ``<dy @ R, x>`` (fp32, ``(1,)``), from the same
    pass when asked for (``x`` is needed then only)."""
    _need_gpu("linear_rbias_bwd_", dx, dy, scale_bias)
    dy = _act(dy)
    sb = _native(scale_bias).to(torch.bfloat16)
    d = _rbias_desc(dy.shape[0], in_f, out_f, seed)
    L = _lib.load()
    with _on(dy.device):
        if not want_scale_bias_grad:
            _lib.check(L.rdb_linear_rbias_bwd(_p(dx), dx.stride(0), None, _p(dy), dy.stride(0), None, 0, _p(sb), ctypes.byref(d), None, 0,
                                              _stream(dy.device)), "rdb_linear_rbias_bwd")
            return None
        x = _act(x)
        ws_bytes = int(L.rdb_linear_workspace_bytes(_lib.RDB_OP_LINEAR_RBIAS_BWD, ctypes.byref(d)))
        ws = _workspace(ws_bytes, dy.device)
        ds = torch.empty((1,), dtype=torch.float32, device=dy.device)
        _lib.check(L.rdb_linear_rbias_bwd(_p(dx), dx.stride(0), _p(ds), _p(dy), dy.stride(0), _p(x), x.stride(0), _p(sb), ctypes.byref(d),
                                          _p(ws), ws_bytes, _stream(dy.device)), "rdb_linear_rbias_bwd")
    return ds


def linear_bwd_dcoef(dy: torch.Tensor, x: torch.Tensor, k: int, coef_rows: int, in_f: int, out_f: int, sO: int, sI: int,
                     seed: int, want_scale_bias_grad: bool = False, algo: int = RDB_ALGO_AUTO):
    """``(dcoef, d_scale_bias)`` in fp32: ``dcoef = (dy.T @ x) . Noise.T`` without storing ``dy.T @ x``."""
    _need_gpu("linear_bwd_dcoef", dy, x)
    dy, x = _act(dy), _act(x)
    if x.dtype != dy.dtype:
        x = x.to(dy.dtype)
    shape = (k,) if coef_rows == 0 else (coef_rows, k)
    dcoef = torch.empty(shape, dtype=torch.float32, device=dy.device)
    dsb = torch.empty((1,), dtype=torch.float32, device=dy.device) if want_scale_bias_grad else None
    d = LinearDesc()
    d.tokens, d.in_f, d.out_f, d.k, d.coef_rows = dy.shape[0], int(in_f), int(out_f), int(k), int(coef_rows)
    d.sO, d.sI, d.seed = int(sO), int(sI), _seed(seed)
    d.act_dtype, d.coef_dtype, d.algo = _DT[dy.dtype], RDB_F32, int(algo)
    L = _lib.load()
    with _on(dy.device):
        ws_bytes = L.rdb_linear_workspace_bytes(RDB_OP_LINEAR_BWD_DCOEF, ctypes.byref(d))
        ws = _workspace(ws_bytes, dy.device)
        rc = L.rdb_linear_bwd_dcoef(_p(dcoef), _p(dsb), _p(dy), dy.stride(0), _p(x), x.stride(0), ctypes.byref(d), _p(ws), ws_bytes,
                                    _stream(dy.device))
    _lib.check(rc, "rdb_linear_bwd_dcoef")
    return dcoef, dsb


# ------------------------------------------------------------------------------------------------ fused linear, projected form
def _proj_desc(tokens, in_f, out_f, k, seed, coef_dtype=torch.bfloat16, act_dtype=torch.bfloat16) -> LinearDesc:
    d = LinearDesc()
    d.tokens, d.in_f, d.out_f, d.k, d.coef_rows = int(tokens), int(in_f), int(out_f), int(k), int(out_f)
    d.sO, d.sI, d.seed = int(in_f), 1, _seed(seed)
    d.act_dtype, d.coef_dtype, d.algo = _DT[act_dtype], _DT[coef_dtype], RDB_ALGO_AUTO
    return d


class _ProjPlan:
    """What the projected calls need to know about a layer and batch, asked of the library once per (sizes, seed)."""
    __slots__ = ("desc", "ref", "state_bytes", "state_cols", "ws_bytes", "ws_bytes_to", "chunks")

    def __init__(self, tokens, in_f, out_f, k, seed, dtype):
        L = _lib.load()
        self.desc = _proj_desc(tokens, in_f, out_f, k, seed, dtype, dtype)
        self.ref = ctypes.byref(self.desc)
        self.state_bytes = int(L.rdb_linear_projection_bytes(self.ref))
        self.state_cols = -(-self.state_bytes // tokens) if self.state_bytes > 0 else 0
        self.ws_bytes = int(L.rdb_linear_workspace_bytes(RDB_OP_LINEAR_BWD_PROJECTED, self.ref))
        self.ws_bytes_to = int(L.rdb_linear_workspace_bytes(_lib.RDB_OP_LINEAR_BWD_PROJECTED_TO, self.ref))
        self.chunks = int(L.rdb_linear_projection_chunks(self.ref, None)) if self.state_bytes > 0 else 0


_plans: dict = {}


def _plan(tokens: int, in_f: int, out_f: int, k: int, seed: int, dtype=torch.bfloat16) -> _ProjPlan:
    key = (tokens, in_f, out_f, k, seed, dtype)
    p = _plans.get(key)
    if p is None:
        if len(_plans) > 4096:
            _plans.clear()
        p = _plans[key] = _ProjPlan(tokens, in_f, out_f, k, _seed(seed), dtype)
    return p


def linear_projection_bytes(tokens: int, in_f: int, out_f: int, k: int, dtype=torch.bfloat16) -> int:
    """Size of the projection state of a layer of these sizes; 0 when the projected form (matrix-coef, bf16 or fp32) does not apply."""
    return int(_lib.load().rdb_linear_projection_bytes(ctypes.byref(_proj_desc(tokens, in_f, out_f, k, 0, dtype, dtype))))


def linear_projection_supported(tokens: int, in_f: int, out_f: int, k: int, dtype=torch.bfloat16) -> bool:
    """Whether the projected entry points run a layer of these sizes: matrix-coef bf16, sizes in multiples of 8 (any number
    of tokens: activations beyond one launch's 2^29 elements are run in chunks of tokens by the library).  Plain integer
    arithmetic, the library's own rule restated (``rdb_linear_projection_bytes(desc) > 0``; a test holds the two together), so
    that a tracing compiler can follow the choice of path without calling into the library."""
    if dtype == torch.float32:   # z in fp32, one launch's worth of tokens, any sizes
        return (min(tokens, in_f, out_f, k) > 0 and tokens * k < (1 << 29) and out_f * k < (1 << 29) and max(in_f, out_f) < (1 << 30)
                and tokens * max(in_f, out_f) < (1 << 28))
    if min(tokens, in_f, out_f, k) <= 0 or k % 8 or in_f % 8 or out_f % 8:
        return False
    kpad, out64 = -(-k // 64) * 64, -(-out_f // 64) * 64
    per_chunk = ((1 << 28) // max(in_f, out_f, kpad)) // 256 * 256   # tokens of one launch
    if per_chunk < 256:
        return False
    nchunks = -(-tokens // per_chunk)
    chunk = -(-(-(-tokens // nchunks)) // 256) * 256 if nchunks > 1 else tokens
    tok64 = -(-chunk // 64) * 64
    limit = 1 << 29   # elements one buffer descriptor addresses
    return tok64 * kpad < limit and out64 * kpad < limit and chunk * k < limit and out_f * k < limit


def linear_projection_preferred(tokens: int, in_f: int, out_f: int, k: int, dtype=torch.bfloat16) -> bool:
    """Whether a training step should save the projection state for its backward pass.  Two conditions.  Speed: the factored
    products need 2*tokens*k*(in_f + out_f) flops per direction, a product on a stored weight 2*tokens*in_f*out_f; the kernels
    that form the weight on chip instead lose against the factored ones up to at least 8 times that (measured), so the bound
    is 16 times, as in the library.  Memory: the state holds z twice (two element orders), 2 * 2 * k bytes per token with k
    rounded up to 64, where the reference's autograd saves the 2 * in_f bytes of x (src/rten_cpp/RandumbTensor.py:942-946);
    the state may cost up to twice that, i.e. k rounded up to 64 must not exceed in_f (768 -> 3072, k = 256: 1024 against
    1536 bytes per token).  Layers that fail the second test still run the factored kernels, through ``rdb_linear_fwd`` and a
    transient workspace, with x saved.  fp32 layers: the state is z in fp32 (4 k bytes per token against 4 in_f)."""
    # not in the few-token regimes, whose vector-ALU kernels (k <= 256 up to 96 tokens; in fp32 also k <= 64 up to 1024 tokens)
    # have no projected form: rdb_linear_fwd and the two gradient calls take them
    few = k * (in_f + out_f) < in_f * out_f and ((dtype == torch.float32 and k <= 64 and tokens <= 1024) or (
        k <= 256 and tokens <= 96 and (k <= 64 or dtype == torch.float32 or max(in_f, out_f) >= 1536)))
    if dtype == torch.float32:
        # the state is z in fp32, 4 k bytes per token where x has 4 in_f: the same memory rule
        return k <= 2 * in_f and not few and (k > 64 or tokens > 1024) and linear_projection_supported(tokens, in_f, out_f, k, dtype)
    kpad = -(-k // 64) * 64
    return (k * (in_f + out_f) < 16 * in_f * out_f and kpad <= in_f and not few
            and linear_projection_supported(tokens, in_f, out_f, k))


def linear_project(x: torch.Tensor, k: int, out_f: int, seed: int, coef: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Projection state of ``x`` for a matrix-coef bf16 layer: an opaque byte tensor ``(tokens, bytes per token)`` holding ``z = x @ Noise.T`` (tokens, k)
    in the element orders the consumers' matrix instructions read (all that the forward product and the coef gradient need
    of ``x``) and, when ``coef`` (out_f, k) is given in bf16, the transposed coefficients for the input gradient."""
    _need_gpu("linear_project", x, coef)
    x = _act(x)
    if x.dtype not in _DT:
        raise ValueError("linear_project computes in bf16 or fp32")
    d = _proj_desc(x.shape[0], x.shape[1], out_f, k, seed, x.dtype, x.dtype)
    L = _lib.load()
    nbytes = L.rdb_linear_projection_bytes(ctypes.byref(d))
    if nbytes <= 0:
        _lib.check(L.rdb_linear_project(None, None, x.stride(0), None, ctypes.byref(d), None), "rdb_linear_project")
    # 2-D so that the token count travels with the tensor: (tokens, bytes per token rounded up)
    state = torch.empty((x.shape[0], -(-nbytes // x.shape[0])), dtype=torch.uint8, device=x.device)
    c = None
    if coef is not None and coef.dtype == torch.bfloat16:
        c = coef.contiguous()
        if tuple(c.shape) != (out_f, k):
            raise ValueError(f"coef must be ({out_f}, {k}), got {tuple(c.shape)}")
    with _on(x.device):
        rc = L.rdb_linear_project(_p(state), _p(x), x.stride(0), _p(c), ctypes.byref(d), _stream(x.device))
    _lib.check(rc, "rdb_linear_project")
    return state


def linear_project_fwd(x: torch.Tensor, coef: torch.Tensor, seed: int, bias: Optional[torch.Tensor] = None):
    """``(y, state)``: :func:`linear_project` (with ``coef``) and :func:`linear_fwd_projected` in one call, for k <= 256 in a
    single kernel launch; the forward pass of a training step, ``state`` being what it saves for backward."""
    if not (x.is_cuda and coef.is_cuda):
        _need_gpu("linear_project_fwd", x, coef)
    x = _act(x)
    c = coef if coef.is_contiguous() else coef.contiguous()
    if x.dtype != c.dtype or x.dtype not in _DT:
        raise ValueError("linear_project_fwd computes in bf16 or in fp32: activations and coefficients in one of them")
    out_f, k = c.shape
    tokens = x.shape[0]
    pl = _plan(tokens, x.shape[1], out_f, k, seed, x.dtype)
    L = _lib.load()
    if pl.state_bytes <= 0:
        _lib.check(L.rdb_linear_project(None, None, x.stride(0), None, pl.ref, None), "rdb_linear_project")
    dev = x.device
    state = torch.empty((tokens, pl.state_cols), dtype=torch.uint8, device=dev)
    b = None if bias is None else bias.to(x.dtype).contiguous()
    y = torch.empty((tokens, out_f), dtype=x.dtype, device=dev)
    with _on(dev):
        st = _stream(dev)
        rc = L.rdb_linear_project_fwd(y.data_ptr(), out_f, state.data_ptr(), x.data_ptr(), x.stride(0), c.data_ptr(),
                                      None if b is None else b.data_ptr(), pl.ref, st)
        if rc:
            _lib.check(rc, "rdb_linear_project_fwd")
        _watch(dev).tick(st)
    return y, state


def projection_unpack(state: torch.Tensor, in_f: int, out_f: int, k: int, dtype=torch.bfloat16) -> dict:
    """The pieces of a projection state as ordinary row-major tensors, for tools and tests (a layout decode, no arithmetic):
    ``z`` (tokens, k) as the forward product reads it, ``z_t`` (k, tokens) as the coef gradient reads it, and ``coef_t``
    (k, out_f), the transposed coefficients, or ``None`` when the state was written without them."""
    tokens = state.shape[0]
    if dtype == torch.float32:   # z row-major in fp32 behind the header; no transposed copies
        d = _proj_desc(tokens, in_f, out_f, k, 0, dtype, dtype)
        _check_state(state, d, "projection_unpack")
        z = state.reshape(-1)[256:256 + 4 * tokens * k].view(torch.float32).view(tokens, k)
        return {"z": z.clone(), "z_t": z.t().contiguous(), "coef_t": None}
    d = _proj_desc(tokens, in_f, out_f, k, 0)
    _check_state(state, d, "projection_unpack")
    info = (ctypes.c_int64 * 8)()
    _lib.check(_lib.load().rdb_linear_projection_layout(ctypes.byref(d), info), "rdb_linear_projection_layout")
    zf_off, frag_fwd, ztf_off, ctf_off, kpad, tok32, tok64, out64 = (int(v) for v in info)
    flat = state.reshape(-1)
    dev = state.device

    def piece(off, nelem):
        return flat[off:off + 2 * nelem].view(torch.bfloat16)

    def frag_gather(buf, rows, kks, ksteps):
        r = torch.arange(rows, device=dev).view(-1, 1)
        c = torch.arange(kks, device=dev).view(1, -1)
        idx = ((r // 32) * ksteps + c // 16) * 512 + (((c // 8) % 2) * 32 + r % 32) * 8 + c % 8
        return buf[idx]

    if frag_fwd:
        z = frag_gather(piece(zf_off, tok32 * kpad), tokens, k, kpad // 16)
    else:
        z = piece(zf_off, tokens * k).view(tokens, k).clone()
    z_t = frag_gather(piece(ztf_off, tok64 * kpad), k, tokens, tok64 // 16)
    has_c = int(flat[:4].view(torch.int32)[0]) == 1
    coef_t = frag_gather(piece(ctf_off, out64 * kpad), k, out_f, out64 // 16) if has_c else None
    return {"z": z, "z_t": z_t, "coef_t": coef_t}


def _check_state(state: torch.Tensor, d: LinearDesc, who: str) -> None:
    need = _lib.load().rdb_linear_projection_bytes(ctypes.byref(d))
    if state.dtype != torch.uint8 or state.dim() != 2 or not state.is_contiguous() or state.numel() < need or need <= 0:
        raise ValueError(f"{who}: the projection state must be the byte tensor linear_project returned for this layer and token "
                         f"count ({need} bytes), got {tuple(state.shape)} {state.dtype}")


def linear_fwd_projected(state: torch.Tensor, coef: torch.Tensor, in_f: int, seed: int,
                         bias: Optional[torch.Tensor] = None, f32_state: bool = False) -> torch.Tensor:
    """``y = z @ coef.T (+ bias)`` for matrix-coef ``coef`` (out_f, k) in bf16; ``state`` from :func:`linear_project`.
    ``f32_state``: the state is that of an fp32 layer (fp32 activations and coefficients)."""
    _need_gpu("linear_fwd_projected", state, coef)
    c = _native(coef)
    out_f, k = c.shape
    tokens = state.shape[0]
    act = torch.float32 if (f32_state and c.dtype == torch.float32) else torch.bfloat16
    d = _proj_desc(tokens, in_f, out_f, k, seed, c.dtype, act)
    _check_state(state, d, "linear_fwd_projected")
    b = None if bias is None else bias.to(act).contiguous()
    y = torch.empty((tokens, out_f), dtype=act, device=state.device)
    with _on(state.device):
        rc = _lib.load().rdb_linear_fwd_projected(_p(y), y.stride(0), _p(state), _p(c), _p(b), ctypes.byref(d), _stream(state.device))
    _lib.check(rc, "rdb_linear_fwd_projected")
    return y


def linear_bwd_dcoef_projected(dy: torch.Tensor, state: torch.Tensor, k: int, in_f: int, seed: int) -> torch.Tensor:
    """``dcoef = dy.T @ z`` (out_f, k) in fp32; ``state`` from :func:`linear_project`."""
    _need_gpu("linear_bwd_dcoef_projected", dy, state)
    dy = _act(dy)
    out_f = dy.shape[1]
    d = _proj_desc(dy.shape[0], in_f, out_f, k, seed)
    _check_state(state, d, "linear_bwd_dcoef_projected")
    dcoef = torch.empty((out_f, k), dtype=torch.float32, device=dy.device)
    with _on(dy.device):
        rc = _lib.load().rdb_linear_bwd_dcoef_projected(_p(dcoef), _p(dy), dy.stride(0), _p(state), ctypes.byref(d), _stream(dy.device))
    _lib.check(rc, "rdb_linear_bwd_dcoef_projected")
    return dcoef


# The backward kernels read C transposed from the copy the forward pass left in the state and never look at the values
# behind ``coef`` for dy.C: a caller that changes coef between the two passes (an optimizer step before a delayed backward,
# a state kept across steps) gets the gradient of the old coefficients with no error.  autograd's version counters catch that
# for tensors it saved; RANDUMB_CHECK_STATE=1 (or this flag) makes every linear_bwd_projected compare the copy with coef
# first, at the price of a device synchronisation.
CHECK_STATE_COEF = os.environ.get("RANDUMB_CHECK_STATE", "0") not in ("", "0")


def check_state_coef(state: torch.Tensor, coef: torch.Tensor, in_f: int) -> None:
    """Raises if the transposed coefficients inside ``state`` are not the values of ``coef`` (out_f, k)."""
    out_f, k = coef.shape
    got = projection_unpack(state, in_f, out_f, k)["coef_t"]
    if got is not None and not torch.equal(got, coef.to(torch.bfloat16).t()):
        raise _lib.RandumbHipError("linear_bwd_projected: the coefficients have changed since the forward pass wrote this projection "
                                   "state; its copy of them is what the backward kernels would read")


def linear_bwd_projected(dy: torch.Tensor, state: torch.Tensor, coef: torch.Tensor, in_f: int, seed: int, ordered_sums: bool = True,
                         dcoef_dtype: torch.dtype = torch.float32, want_dx: bool = True):
    """Whole backward pass of a matrix-coef layer from the projection state: ``(dx, dcoef)`` with ``dx = dy @ W`` in the
    activations' dtype and ``dcoef = dy.T @ z``, in two kernel launches for bf16.  ``ordered_sums`` gives the library room for
    the partial sums of ``dcoef`` (added in a fixed order: bit-reproducible); without it (bf16 only) they are combined with
    fp32 atomics.  ``dcoef_dtype``: fp32, or bf16 to have the sums rounded once by the kernel that adds them up (what
    ``.to(bfloat16)`` would give, without the extra pass; layers whose tokens the library runs in several chunks get fp32 sums
    rounded by torch instead).  fp32 layers (``dy`` and ``coef`` in fp32): sums in fp32 in a fixed order; ``want_dx=False``
    returns ``(None, dcoef)``."""
    if not (dy.is_cuda and state.is_cuda and coef.is_cuda):
        _need_gpu("linear_bwd_projected", dy, state, coef)
    dy = _act(dy)
    c = _native(coef)
    out_f, k = c.shape
    tokens = dy.shape[0]
    f32 = dy.dtype == torch.float32 and c.dtype == torch.float32
    pl = _plan(tokens, in_f, out_f, k, seed, torch.float32 if f32 else torch.bfloat16)
    if not f32 and c.dtype != torch.bfloat16:
        _check_state(state, _proj_desc(tokens, in_f, out_f, k, seed, c.dtype), "linear_bwd_projected")
    elif state.dtype != torch.uint8 or state.dim() != 2 or state.numel() < pl.state_bytes or pl.state_bytes <= 0 or not state.is_contiguous():
        _check_state(state, pl.desc, "linear_bwd_projected")
    if CHECK_STATE_COEF and not f32:
        check_state_coef(state, c, in_f)
    if dcoef_dtype not in (torch.float32, torch.bfloat16):
        raise ValueError("dcoef_dtype must be float32 or bfloat16")
    if not want_dx and not f32:
        raise ValueError("want_dx=False is for fp32 layers; bf16 layers have linear_bwd_dcoef_projected")
    in_kernel = dcoef_dtype == torch.bfloat16 and ordered_sums and pl.chunks == 1 and c.dtype == torch.bfloat16
    dev = dy.device
    dx = torch.empty((tokens, in_f), dtype=dy.dtype, device=dev) if want_dx else None
    dcoef = torch.empty((out_f, k), dtype=torch.bfloat16 if in_kernel else torch.float32, device=dev)
    L = _lib.load()
    d = pl.desc if (f32 or c.dtype == torch.bfloat16) else _proj_desc(tokens, in_f, out_f, k, seed, c.dtype)
    ref = pl.ref if d is pl.desc else ctypes.byref(d)
    with _on(dev):
        if in_kernel:
            ws_bytes = pl.ws_bytes_to
        elif ordered_sums or f32:
            ws_bytes = pl.ws_bytes
        else:
            ws_bytes = int(L.rdb_linear_workspace_bytes(RDB_OP_LINEAR_BWD_DX, ref))
        ws = _workspace(ws_bytes, dev)
        st = _stream(dev)
        if in_kernel:
            rc = L.rdb_linear_bwd_projected_to(dx.data_ptr(), in_f, dcoef.data_ptr(), RDB_BF16, dy.data_ptr(), dy.stride(0), state.data_ptr(),
                                               c.data_ptr(), ref, _p(ws), ws_bytes, st)
        else:
            rc = L.rdb_linear_bwd_projected(None if dx is None else dx.data_ptr(), in_f, dcoef.data_ptr(), dy.data_ptr(), dy.stride(0),
                                            state.data_ptr(), c.data_ptr(), ref, _p(ws), ws_bytes, st)
    if rc:
        _lib.check(rc, "rdb_linear_bwd_projected")
    return dx, (dcoef if dcoef.dtype == dcoef_dtype else dcoef.to(dcoef_dtype))


def set_f32_split(mode: int) -> int:
    """Process-wide switch of the fp32 products that run on the matrix cores: 1 (default) = three-way bf16 splits of the operands
    and six bf16 matrix instructions per product (fp32 accuracy at 3/8 of the matrix-core time), 0 = fp32 matrix instructions.
    Returns the previous mode."""
    return int(_lib.load().rdb_set_f32_split(int(mode)))


def set_big_tiles(mode: int) -> int:
    """Process-wide switch of the projected entry points' kernels for k > 256: 0 = 128-wide tiles only, 1 = 256-wide tiles
    (one persistent block per compute unit) when the layer has a tile for every other compute unit at least (default),
    2 = 256-wide tiles whenever k > 256.  y and dx are the same bit for bit either way, dcoef up to the order of fp32 sums over
    token ranges.  Returns the previous mode."""
    return int(_lib.load().rdb_set_big_tiles(int(mode)))
