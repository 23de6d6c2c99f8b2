"""ctypes binding of ``librandumb_hip.so`` (the C ABI declared in ``include/randumb_hip.h``).

The library is the only compute path of this package: if it has not been built the loader raises, it never
falls back to another implementation.  Build it with ``make -C randumb_amd/csrc`` (or
``python -c "import __graft_entry__ as g; g.build()"`` from the repository root).
"""
from __future__ import annotations

import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
SO_PATH = os.path.join(_HERE, "librandumb_hip.so")

RDB_F32, RDB_BF16 = 0, 1
RDB_ALGO_AUTO, RDB_ALGO_TILE, RDB_ALGO_STRIP, RDB_ALGO_FACTORED = 0, 1, 2, 3
RDB_OP_LINEAR_FWD, RDB_OP_LINEAR_BWD_DX, RDB_OP_LINEAR_BWD_DCOEF, RDB_OP_LINEAR_BWD_PROJECTED, RDB_OP_LINEAR_BWD_PROJECTED_TO = 0, 1, 2, 3, 4
RDB_OP_LINEAR_BWD_DX_DSCALE = 5
RDB_OP_LINEAR_RBIAS_BWD = 6

# every exported entry point, in header order; tests check the list against the built library
EXPORTS = [
    "rdb_abi_version",
    "rdb_last_error_string",
    "rdb_sq5_fill_2d",
    "rdb_sq5_fill_1d",
    "rdb_materialize_fwd",
    "rdb_materialize_bwd",
    "rdb_materialize_bwd_workspace_bytes",
    "rdb_scale_bias_bwd",
    "rdb_scale_bias_bwd_workspace_bytes",
    "rdb_embed_fwd",
    "rdb_embed_bwd",
    "rdb_embed_bwd_workspace_bytes",
    "rdb_linear_workspace_bytes",
    "rdb_linear_fwd",
    "rdb_linear_fwd_static",
    "rdb_linear_fwd_static_max_bytes",
    "rdb_linear_bwd_dx",
    "rdb_linear_bwd_dx_dscale",
    "rdb_linear_rbias_fwd",
    "rdb_linear_rbias_bwd",
    "rdb_linear_bwd_dcoef",
    "rdb_linear_projection_bytes",
    "rdb_linear_projection_chunks",
    "rdb_linear_projection_layout",
    "rdb_linear_project",
    "rdb_linear_project_fwd",
    "rdb_linear_fwd_projected",
    "rdb_linear_bwd_dcoef_projected",
    "rdb_linear_bwd_projected",
    "rdb_linear_bwd_projected_to",
    "rdb_linear_bwd_projected_part",
    "rdb_set_big_tiles",
    "rdb_set_f32_split",
    "rdb_set_one_launch",
    "rdb_sync_giveups_async",
    "rdb_sync_giveups",
    "rdb_selftest_sync_giveup",
]

ABI_VERSION = 8   # what this binding was written against (rdb_abi_version)


class LinearDesc(ctypes.Structure):
    """Mirror of ``rdb_linear_desc``."""

    _fields_ = [
        ("tokens", ctypes.c_int64),
        ("in_f", ctypes.c_int64),
        ("out_f", ctypes.c_int64),
        ("k", ctypes.c_int64),
        ("coef_rows", ctypes.c_int64),
        ("sO", ctypes.c_int64),
        ("sI", ctypes.c_int64),
        ("seed", ctypes.c_uint32),
        ("act_dtype", ctypes.c_int32),
        ("coef_dtype", ctypes.c_int32),
        ("algo", ctypes.c_int32),
    ]


class RandumbHipError(RuntimeError):
    pass


_lib = None


def load() -> ctypes.CDLL:
    """Loads the shared library once; raises if it is missing (there is no fallback path)."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(SO_PATH):
        raise RandumbHipError(
            f"{SO_PATH} is missing: build it with `make -C randumb_amd/csrc` "
            "(hipcc, --offload-arch=gfx950). randumb_amd has no other compute path."
        )
    L = ctypes.CDLL(SO_PATH)
    i64, u32, vp, ci = ctypes.c_int64, ctypes.c_uint32, ctypes.c_void_p, ctypes.c_int
    L.rdb_abi_version.restype = ci
    L.rdb_abi_version.argtypes = []
    # a library built from other sources may export the same names with other argument lists: calling those with this
    # binding's arguments would hand the kernels shifted pointers
    found = int(L.rdb_abi_version())
    if found != ABI_VERSION:
        raise RandumbHipError(f"{SO_PATH} has ABI version {found}, this package binds version {ABI_VERSION}: rebuild it with "
                              "`make -C randumb_amd/csrc`")
    L.rdb_last_error_string.restype = ctypes.c_char_p
    L.rdb_last_error_string.argtypes = []
    L.rdb_sq5_fill_2d.argtypes = [vp, i64, i64, u32, vp]
    L.rdb_sq5_fill_1d.argtypes = [vp, i64, u32, vp]
    L.rdb_materialize_fwd.argtypes = [vp, vp, ci, i64, i64, i64, i64, i64, i64, i64, u32, vp, vp]
    L.rdb_materialize_bwd.argtypes = [vp, vp, ci, i64, i64, i64, i64, u32, vp, i64, vp]
    L.rdb_materialize_bwd_workspace_bytes.argtypes = [i64, i64, i64, i64]
    L.rdb_materialize_bwd_workspace_bytes.restype = i64
    L.rdb_scale_bias_bwd.argtypes = [vp, vp, ci, i64, u32, vp, i64, vp]
    L.rdb_scale_bias_bwd_workspace_bytes.argtypes = [i64]
    L.rdb_scale_bias_bwd_workspace_bytes.restype = i64
    L.rdb_embed_fwd.argtypes = [vp, vp, i64, vp, ci, i64, i64, u32, vp]
    L.rdb_embed_bwd.argtypes = [vp, vp, i64, vp, ci, i64, i64, u32, vp, i64, vp]
    L.rdb_embed_bwd_workspace_bytes.argtypes = [i64, i64, i64]
    L.rdb_embed_bwd_workspace_bytes.restype = i64
    dp = ctypes.POINTER(LinearDesc)
    L.rdb_linear_workspace_bytes.argtypes = [ci, dp]
    L.rdb_linear_workspace_bytes.restype = i64
    L.rdb_linear_fwd.argtypes = [vp, i64, vp, i64, vp, vp, vp, dp, vp, i64, vp]
    L.rdb_linear_fwd_static.argtypes = [vp, i64, vp, i64, vp, vp, vp, dp, vp]
    L.rdb_linear_fwd_static.restype = ci
    L.rdb_linear_fwd_static_max_bytes.argtypes = []
    L.rdb_linear_fwd_static_max_bytes.restype = i64
    L.rdb_linear_bwd_dx.argtypes = [vp, i64, vp, i64, vp, vp, dp, vp, i64, vp]
    L.rdb_linear_bwd_dcoef.argtypes = [vp, vp, vp, i64, vp, i64, dp, vp, i64, vp]
    L.rdb_linear_bwd_dx_dscale.argtypes = [vp, i64, vp, vp, i64, vp, i64, vp, vp, dp, vp, i64, vp]
    L.rdb_linear_rbias_fwd.argtypes = [vp, i64, vp, i64, vp, dp, vp]
    L.rdb_linear_rbias_bwd.argtypes = [vp, i64, vp, vp, i64, vp, i64, vp, dp, vp, i64, vp]
    L.rdb_linear_projection_bytes.argtypes = [dp]
    L.rdb_linear_projection_bytes.restype = i64
    L.rdb_linear_projection_chunks.argtypes = [dp, ctypes.POINTER(i64)]
    L.rdb_linear_projection_chunks.restype = ci
    L.rdb_linear_projection_layout.argtypes = [dp, ctypes.POINTER(i64)]
    L.rdb_linear_projection_layout.restype = ci
    L.rdb_linear_project.argtypes = [vp, vp, i64, vp, dp, vp]
    L.rdb_linear_project_fwd.argtypes = [vp, i64, vp, vp, i64, vp, vp, dp, vp]
    L.rdb_linear_fwd_projected.argtypes = [vp, i64, vp, vp, vp, dp, vp]
    L.rdb_linear_bwd_dcoef_projected.argtypes = [vp, vp, i64, vp, dp, vp]
    L.rdb_linear_bwd_projected.argtypes = [vp, i64, vp, vp, i64, vp, vp, dp, vp, i64, vp]
    L.rdb_linear_bwd_projected_to.argtypes = [vp, i64, vp, ci, vp, i64, vp, vp, dp, vp, i64, vp]
    L.rdb_linear_bwd_projected_part.argtypes = [ci, vp, i64, vp, vp, i64, vp, vp, dp, vp, i64, vp]
    L.rdb_set_big_tiles.argtypes = [ci]
    L.rdb_set_big_tiles.restype = ci
    L.rdb_set_f32_split.argtypes = [ci]
    L.rdb_set_f32_split.restype = ci
    L.rdb_set_one_launch.argtypes = [ci]
    L.rdb_set_one_launch.restype = ci
    L.rdb_sync_giveups_async.argtypes = [vp, vp]
    L.rdb_sync_giveups_async.restype = ci
    L.rdb_sync_giveups.argtypes = [vp, vp]
    L.rdb_sync_giveups.restype = ci
    L.rdb_selftest_sync_giveup.argtypes = [vp, i64, vp, i64, vp, dp, ci, vp]
    L.rdb_selftest_sync_giveup.restype = ci
    for name in ("rdb_sq5_fill_2d", "rdb_sq5_fill_1d", "rdb_materialize_fwd", "rdb_materialize_bwd", "rdb_scale_bias_bwd",
                 "rdb_embed_fwd", "rdb_embed_bwd", "rdb_linear_fwd", "rdb_linear_bwd_dx", "rdb_linear_bwd_dx_dscale", "rdb_linear_rbias_fwd",
                 "rdb_linear_rbias_bwd", "rdb_linear_bwd_dcoef",
                 "rdb_linear_project", "rdb_linear_project_fwd", "rdb_linear_fwd_projected", "rdb_linear_bwd_dcoef_projected",
                 "rdb_linear_bwd_projected", "rdb_linear_bwd_projected_to", "rdb_linear_bwd_projected_part"):
        getattr(L, name).restype = ci
    _lib = L
    return L


def check(rc: int, what: str) -> None:
    """Turns a non-zero return code into an exception carrying the library's message."""
    if rc != 0:
        msg = load().rdb_last_error_string().decode("utf-8", "replace")
        kind = "argument error" if rc < 0 else "HIP error"
        raise RandumbHipError(f"{what}: {kind} {rc}: {msg}")
