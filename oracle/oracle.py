"""CPU oracle for the RANDUMB pseudorandom-matrix hot path (TEST INFRASTRUCTURE ONLY).

Only tests, the smoke check and the benchmark's CPU-baseline leg may import this
module; the shipped package never does.  It restates the reference arithmetic three
independent ways so that a slip in one spelling is caught by the others:

* ``sq5_u32_py``     - arbitrary-precision Python integers with an explicit 2**32 mask
* ``sq5_u32_np``     - NumPy ``uint32`` vector arithmetic (wraps natively)
* ``librdb_oracle``  - plain C ``uint32_t`` (``rdb_oracle.c``), loaded through ctypes

Reference citations (paths relative to the reference checkout):
``R.py`` = ``src/rten_cpp/RandumbTensor.py``, ``R.cu`` = ``src/rten_cpp/csrc/cuda/rten.cu``.
"""
from __future__ import annotations

import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "librdb_oracle.so")

SQ5_BIT_NOISE1 = 0xD2A80A3F
SQ5_BIT_NOISE2 = 0xA884F197
SQ5_BIT_NOISE3 = 0x6C736F4B
SQ5_BIT_NOISE4 = 0xB79F3ABB
SQ5_BIT_NOISE5 = 0x1B56C4F5
PRIME = 198491317
_MASK = 0xFFFFFFFF


# ----------------------------------------------------------------------------- pure Python
def sq5_u32_py(idx: int, seed: int) -> int:
    """Squirrel5 mangle on Python ints.  R.py:148-159 / R.py:216-227 / R.cu:33-44."""
    b = idx & _MASK
    b = (b * SQ5_BIT_NOISE1) & _MASK
    b = (b + seed) & _MASK
    b ^= b >> 9
    b = (b + SQ5_BIT_NOISE2) & _MASK
    b ^= b >> 11
    b = (b * SQ5_BIT_NOISE3) & _MASK
    b ^= b >> 13
    b = (b + SQ5_BIT_NOISE4) & _MASK
    b ^= b >> 15
    b = (b * SQ5_BIT_NOISE5) & _MASK
    b ^= b >> 17
    return b


def u32_to_f32_py(bits: int) -> float:
    """int32 reinterpretation -> fp32 (RNE) -> times 2**-31.  R.py:162-163, R.cu:19,47."""
    s = bits - (1 << 32) if bits & 0x80000000 else bits
    return float(np.float32(s) * np.float32(2.0 ** -31))


def mix2d_py(n: int, m: int) -> int:
    """Noise address of row ``n`` (tensor element) and column ``m`` (coef index).  R.py:148."""
    return (PRIME * n + m) & _MASK


def noise_py(n: int, m: int, seed: int) -> float:
    return u32_to_f32_py(sq5_u32_py(mix2d_py(n, m), seed))


# ----------------------------------------------------------------------------- NumPy
def sq5_u32_np(idx, seed: int) -> np.ndarray:
    """Vectorised Squirrel5 on ``uint32`` arrays (wrap-around is the dtype's own)."""
    with np.errstate(over="ignore"):
        b = np.asarray(idx).astype(np.uint32, copy=True)
        b *= np.uint32(SQ5_BIT_NOISE1)
        b += np.uint32(seed & _MASK)
        b ^= b >> np.uint32(9)
        b += np.uint32(SQ5_BIT_NOISE2)
        b ^= b >> np.uint32(11)
        b *= np.uint32(SQ5_BIT_NOISE3)
        b ^= b >> np.uint32(13)
        b += np.uint32(SQ5_BIT_NOISE4)
        b ^= b >> np.uint32(15)
        b *= np.uint32(SQ5_BIT_NOISE5)
        b ^= b >> np.uint32(17)
    return b


def u32_to_f32_np(bits: np.ndarray) -> np.ndarray:
    return bits.view(np.int32).astype(np.float32) * np.float32(2.0 ** -31)


def noise_1d_np(idx, seed: int) -> np.ndarray:
    """R.py:204-232."""
    return u32_to_f32_np(sq5_u32_np(idx, seed))


def noise_2d_np(rows, cols, seed: int) -> np.ndarray:
    """Tile ``[len(rows), len(cols)]`` of the noise matrix.  R.py:130-164."""
    with np.errstate(over="ignore"):
        r = np.asarray(rows).astype(np.uint32) * np.uint32(PRIME)
        a = r[:, None] + np.asarray(cols).astype(np.uint32)[None, :]
    return u32_to_f32_np(sq5_u32_np(a, seed))


def materialize_fwd_np(coef: np.ndarray, size, strides, seed: int, scale_bias=None,
                       row_len: int | None = None) -> np.ndarray:
    """Dense fp64 ``Noise @ c`` restatement of R.py:235-290 (brute force; small shapes only).

    ``coef.ndim == 1``: vector-coef form.  ``coef.ndim == 2``: matrix-coef form over a contiguous
    ``(coef.shape[0], row_len)`` base tensor.
    """
    size = tuple(size)
    strides = tuple(strides)
    if len(size) == 1:  # R.py:375-377
        size, strides = (1, size[0]), (0, strides[0])
    P, Q = size
    n = np.arange(P * Q, dtype=np.int64)
    a = (n % Q) * strides[1] + (n // Q) * strides[0]  # R.py:264
    coef = np.asarray(coef)
    if coef.ndim == 1:
        k = coef.shape[0]
        noise = noise_2d_np(a, np.arange(k), seed).astype(np.float64)
        out = noise @ coef.astype(np.float64)
    else:
        assert row_len is not None
        k = coef.shape[1]
        noise = noise_2d_np(a % row_len, np.arange(k), seed).astype(np.float64)
        out = np.einsum("nm,nm->n", noise, coef.astype(np.float64)[a // row_len])
    if scale_bias is not None:  # R.py:286-289
        out = out + float(scale_bias) * noise_1d_np(a, seed).astype(np.float64)
    return out.reshape(P, Q)


def materialize_bwd_np(dW: np.ndarray, k: int, seed: int, coef_rows: int = 0) -> np.ndarray:
    """Dense fp64 ``Noise.T @ dW`` restatement of R.py:304-359."""
    d = np.asarray(dW, dtype=np.float64)
    if coef_rows == 0:
        d = d.reshape(-1)
        noise = noise_2d_np(np.arange(d.size), np.arange(k), seed).astype(np.float64)
        return noise.T @ d
    d = d.reshape(coef_rows, -1)
    noise = noise_2d_np(np.arange(d.shape[1]), np.arange(k), seed).astype(np.float64)  # [in, k]
    return d @ noise


# ----------------------------------------------------------------------------- C library
def build(force: bool = False) -> str:
    """Compile ``rdb_oracle.c`` with gcc (idempotent unless ``force``)."""
    src = os.path.join(_HERE, "rdb_oracle.c")
    if force or not os.path.exists(_SO) or os.path.getmtime(_SO) < os.path.getmtime(src):
        subprocess.check_call(["make", "-C", _HERE, "-B", "librdb_oracle.so"],
                              stdout=subprocess.DEVNULL)
    return _SO


_lib = None


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(_SO):
            build()
        L = ctypes.CDLL(_SO)
        i64, u32, fp = ctypes.c_int64, ctypes.c_uint32, ctypes.c_void_p
        L.rdbo_sq5_u32.restype = u32
        L.rdbo_sq5_u32.argtypes = [u32, u32]
        L.rdbo_sq5_f32.restype = ctypes.c_float
        L.rdbo_sq5_f32.argtypes = [u32, u32]
        L.rdbo_noise_at.restype = ctypes.c_float
        L.rdbo_noise_at.argtypes = [u32, u32, u32]
        L.rdbo_noise_2d.argtypes = [fp, i64, i64, u32]
        L.rdbo_noise_1d.argtypes = [fp, i64, u32]
        L.rdbo_materialize_fwd.argtypes = [fp, fp, i64, i64, i64, i64, i64, i64, i64, u32, fp, ctypes.c_int]
        L.rdbo_materialize_bwd.argtypes = [fp, fp, i64, i64, i64, i64, u32]
        L.rdbo_scale_bias_bwd.argtypes = [fp, fp, i64, u32]
        L.rdbo_embed_fwd.argtypes = [fp, fp, i64, fp, i64, i64, u32]
        L.rdbo_embed_bwd.argtypes = [fp, fp, i64, fp, i64, i64, u32]
        L.rdbo_num_threads.restype = ctypes.c_int
        for name in ("rdbo_noise_2d", "rdbo_noise_1d", "rdbo_materialize_fwd", "rdbo_materialize_bwd",
                     "rdbo_scale_bias_bwd", "rdbo_embed_fwd", "rdbo_embed_bwd"):
            getattr(L, name).restype = None
        _lib = L
    return _lib


def _p(a: np.ndarray):
    return a.ctypes.data_as(ctypes.c_void_p)


def _f32(a) -> np.ndarray:
    return np.ascontiguousarray(np.asarray(a, dtype=np.float32))


def noise_2d(N: int, M: int, seed: int) -> np.ndarray:
    out = np.empty((N, M), dtype=np.float32)
    lib().rdbo_noise_2d(_p(out), N, M, seed & _MASK)
    return out


def noise_1d(N: int, seed: int) -> np.ndarray:
    out = np.empty((N,), dtype=np.float32)
    lib().rdbo_noise_1d(_p(out), N, seed & _MASK)
    return out


def materialize_fwd(coef, size, strides, seed: int, scale_bias=None, row_len: int | None = None,
                    acc_double: bool = True) -> np.ndarray:
    """fp32 output of shape ``size``; mirrors op ``rten::materialize_fwd`` (R.py:371-381)."""
    coef = _f32(coef)
    size, strides = tuple(size), tuple(strides)
    out_shape = size
    if len(size) == 1:
        size, strides = (1, size[0]), (0, strides[0])
    P, Q = size
    rows, k = (0, coef.shape[0]) if coef.ndim == 1 else coef.shape
    if coef.ndim == 2:
        assert row_len is not None
    out = np.empty((P * Q,), dtype=np.float32)
    sb = None if scale_bias is None else _f32([float(scale_bias)])
    lib().rdbo_materialize_fwd(_p(out), _p(coef), rows, k, row_len or 0, P, Q, strides[0], strides[1],
                               seed & _MASK, None if sb is None else _p(sb), int(acc_double))
    return out.reshape(out_shape)


def materialize_bwd(dW, k: int, seed: int, coef_rows: int = 0) -> np.ndarray:
    """Mirrors op ``rten::materialize_bwd`` (R.py:383-390); matrix-coef form returns ``(coef_rows, k)``."""
    d = _f32(dW).reshape(-1)
    if coef_rows == 0:
        out = np.empty((k,), dtype=np.float32)
        lib().rdbo_materialize_bwd(_p(out), _p(d), 0, k, 0, d.size, seed & _MASK)
        return out
    out = np.empty((coef_rows, k), dtype=np.float32)
    lib().rdbo_materialize_bwd(_p(out), _p(d), coef_rows, k, d.size // coef_rows, d.size, seed & _MASK)
    return out


def scale_bias_bwd(dW, seed: int) -> np.ndarray:
    d = _f32(dW).reshape(-1)
    out = np.empty((1,), dtype=np.float32)
    lib().rdbo_scale_bias_bwd(_p(out), _p(d), d.size, seed & _MASK)
    return out


def embed_fwd(idx, coef, rowsize: int, seed: int) -> np.ndarray:
    idx = np.ascontiguousarray(np.asarray(idx, dtype=np.int64))
    coef = _f32(coef)
    out = np.empty(idx.shape + (rowsize,), dtype=np.float32)
    lib().rdbo_embed_fwd(_p(out), _p(idx), idx.size, _p(coef), coef.size, rowsize, seed & _MASK)
    return out


def embed_bwd(idx, dout, k: int, rowsize: int, seed: int) -> np.ndarray:
    idx = np.ascontiguousarray(np.asarray(idx, dtype=np.int64))
    d = _f32(dout).reshape(-1)
    out = np.empty((k,), dtype=np.float32)
    lib().rdbo_embed_bwd(_p(out), _p(idx), idx.size, _p(d), k, rowsize, seed & _MASK)
    return out


# ----------------------------------------------------------------------------- linear layer (materialise-then-matmul)
def linear_fwd(x, coef, in_features: int, out_features: int, seed: int, bias=None,
               scale_bias=None) -> np.ndarray:
    """``y = x @ W.T (+ bias)`` on the materialised weight, fp64 matmul.  R.py:771-791, 942-946."""
    coef = np.asarray(coef)
    W = materialize_fwd(coef, (out_features, in_features), (in_features, 1), seed, scale_bias,
                        row_len=in_features if coef.ndim == 2 else None).astype(np.float64)
    y = np.asarray(x, dtype=np.float64) @ W.T
    if bias is not None:
        y = y + np.asarray(bias, dtype=np.float64)
    return y


def linear_bwd(x, dy, coef, in_features: int, out_features: int, seed: int, scale_bias=None):
    """Returns ``(dx, dcoef, dW)`` in fp64/fp32: dx = dy @ W, dW = dy.T @ x, dcoef = Noise.T dW.

    Mirrors autograd's ``MmBackward`` on the materialised weight followed by
    ``RandumbTensorConstructor.backward`` (R.py:979-990).
    """
    coef = np.asarray(coef)
    W = materialize_fwd(coef, (out_features, in_features), (in_features, 1), seed, scale_bias,
                        row_len=in_features if coef.ndim == 2 else None).astype(np.float64)
    x64 = np.asarray(x, dtype=np.float64)
    dy64 = np.asarray(dy, dtype=np.float64)
    dx = dy64 @ W
    dW = dy64.T @ x64
    k = coef.shape[-1]
    dcoef = materialize_bwd_np(dW, k, seed, coef_rows=0 if coef.ndim == 1 else coef.shape[0])
    return dx, dcoef, dW
