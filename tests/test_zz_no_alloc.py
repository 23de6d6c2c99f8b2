"""The entry point that allocates nothing (rdb_linear_fwd_static) against rdb_linear_fwd, through the C ABI."""
import ctypes

import pytest
import torch

from randumb_amd import _lib

pytestmark = pytest.mark.gpu


def _desc(tokens, in_f, out_f, k, seed):
    d = _lib.LinearDesc()
    d.tokens, d.in_f, d.out_f, d.k, d.coef_rows, d.sO, d.sI, d.seed = tokens, in_f, out_f, k, out_f, in_f, 1, seed
    d.act_dtype, d.coef_dtype, d.algo = _lib.RDB_BF16, _lib.RDB_BF16, _lib.RDB_ALGO_AUTO
    return d


def _both(L, tokens, in_f, out_f, k, seed, with_bias):
    g = torch.Generator().manual_seed(1000 + tokens)
    x = torch.randn(tokens, in_f, generator=g).bfloat16().cuda()
    C = (torch.randn(out_f, k, generator=g) * 0.05).bfloat16().cuda()
    bias = torch.randn(out_f, generator=g).bfloat16().cuda() if with_bias else None
    d = _desc(tokens, in_f, out_f, k, seed)
    r = ctypes.byref(d)
    vp = ctypes.c_void_p
    stream = vp(torch.cuda.current_stream().cuda_stream)
    pb = None if bias is None else vp(bias.data_ptr())
    # the existing entry point, scratch in a workspace of the caller's
    n = L.rdb_linear_workspace_bytes(_lib.RDB_OP_LINEAR_FWD, r)
    assert 0 < n <= L.rdb_linear_fwd_static_max_bytes()
    ws = torch.empty(n, dtype=torch.uint8, device="cuda")
    y_ref = torch.full((tokens, out_f), float("nan"), dtype=torch.bfloat16, device="cuda")
    _lib.check(L.rdb_linear_fwd(vp(y_ref.data_ptr()), out_f, vp(x.data_ptr()), in_f, vp(C.data_ptr()), None, pb, r, vp(ws.data_ptr()), n, stream),
               "rdb_linear_fwd")
    # the same request with the scratch in the library's static array
    y = torch.full((tokens, out_f), float("nan"), dtype=torch.bfloat16, device="cuda")
    torch.cuda.synchronize()
    before = torch.cuda.memory_allocated()
    _lib.check(L.rdb_linear_fwd_static(vp(y.data_ptr()), out_f, vp(x.data_ptr()), in_f, vp(C.data_ptr()), None, pb, r, stream), "rdb_linear_fwd_static")
    torch.cuda.synchronize()
    assert torch.cuda.memory_allocated() == before
    return y, y_ref


def test_static_scratch_forward_matches_the_workspace_forward():
    L = _lib.load()
    print("case static scratch, 1024 tokens then 200", flush=True)
    y, y_ref = _both(L, 1024, 768, 512, 256, 3, True)
    assert torch.equal(y, y_ref) and bool(torch.isfinite(y.float()).all())
    # a second, smaller call finds the array full of the first call's state: it must not read any of it
    y, y_ref = _both(L, 200, 768, 512, 256, 4, False)
    assert torch.equal(y, y_ref) and bool(torch.isfinite(y.float()).all())


def test_static_scratch_rejects_what_does_not_fit():
    L = _lib.load()
    d = _desc(65536, 768, 3072, 256, 0)     # 64 MiB of projection state
    rc = L.rdb_linear_fwd_static(ctypes.c_void_p(256), 3072, ctypes.c_void_p(256), 768, ctypes.c_void_p(256), None, None, ctypes.byref(d), None)
    assert rc == -6 and b"static scratch holds" in L.rdb_last_error_string()
