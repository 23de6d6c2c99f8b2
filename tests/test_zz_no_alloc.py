"""The entry point that allocates nothing (rdb_linear_fwd_static) against rdb_linear_fwd, through the C ABI."""
import ctypes

import pytest
import torch

from randumb_amd import _lib

pytestmark = pytest.mark.gpu


def _desc(tokens, in_f, out_f, k, seed, dtype=torch.bfloat16):
    d = _lib.LinearDesc()
    d.tokens, d.in_f, d.out_f, d.k, d.coef_rows, d.sO, d.sI, d.seed = tokens, in_f, out_f, k, out_f, in_f, 1, seed
    code = _lib.RDB_BF16 if dtype == torch.bfloat16 else _lib.RDB_F32
    d.act_dtype, d.coef_dtype, d.algo = code, code, _lib.RDB_ALGO_AUTO
    return d


def _both(L, tokens, in_f, out_f, k, seed, with_bias, dtype=torch.bfloat16, with_scale_bias=False):
    g = torch.Generator().manual_seed(1000 + tokens)
    x = torch.randn(tokens, in_f, generator=g).to(dtype).cuda()
    C = (torch.randn(out_f, k, generator=g) * 0.05).to(dtype).cuda()
    bias = torch.randn(out_f, generator=g).to(dtype).cuda() if with_bias else None
    sb = torch.full((1,), 0.03).to(dtype).cuda() if with_scale_bias else None
    d = _desc(tokens, in_f, out_f, k, seed, dtype)
    r = ctypes.byref(d)
    vp = ctypes.c_void_p
    stream = vp(torch.cuda.current_stream().cuda_stream)
    pb = None if bias is None else vp(bias.data_ptr())
    psb = None if sb is None else vp(sb.data_ptr())
    # the existing entry point, scratch in a workspace of the caller's
    n = L.rdb_linear_workspace_bytes(_lib.RDB_OP_LINEAR_FWD, r)
    assert 0 < n <= L.rdb_linear_fwd_static_max_bytes()
    ws = torch.empty(n, dtype=torch.uint8, device="cuda")
    y_ref = torch.full((tokens, out_f), float("nan"), dtype=dtype, device="cuda")
    _lib.check(L.rdb_linear_fwd(vp(y_ref.data_ptr()), out_f, vp(x.data_ptr()), in_f, vp(C.data_ptr()), psb, pb, r, vp(ws.data_ptr()), n, stream),
               "rdb_linear_fwd")
    # the same request with the scratch in the library's static array
    y = torch.full((tokens, out_f), float("nan"), dtype=dtype, device="cuda")
    torch.cuda.synchronize()
    # torch's own counter sees only torch's allocator; the device's free memory sees a hipMalloc by anybody in the process
    before, free_before = torch.cuda.memory_allocated(), torch.cuda.mem_get_info()[0]
    _lib.check(L.rdb_linear_fwd_static(vp(y.data_ptr()), out_f, vp(x.data_ptr()), in_f, vp(C.data_ptr()), psb, pb, r, stream), "rdb_linear_fwd_static")
    torch.cuda.synchronize()
    assert torch.cuda.memory_allocated() == before
    assert _STATE["warm"] is False or torch.cuda.mem_get_info()[0] == free_before, "the device's free memory changed across the call"
    _STATE["warm"] = True   # the first call of a process may load the library's code object onto the device
    return y, y_ref


_STATE = {"warm": False}


def test_static_scratch_forward_matches_the_workspace_forward():
    L = _lib.load()
    print("case static scratch, 1024 tokens then 200", flush=True)
    y, y_ref = _both(L, 1024, 768, 512, 256, 3, True)
    assert torch.equal(y, y_ref) and bool(torch.isfinite(y.float()).all())
    # a second, smaller call finds the array full of the first call's state: it must not read any of it
    y, y_ref = _both(L, 200, 768, 512, 256, 4, False)
    assert torch.equal(y, y_ref) and bool(torch.isfinite(y.float()).all())


def test_static_scratch_in_fp32_and_with_the_fused_random_bias():
    """The other kernel families that keep scratch in the shared array, back to back on what the previous one left there: the
    fp32 small-k kernels (partial sums and tag slots), the fp32 matrix-core kernels (partial sums over contraction ranges),
    the fp32 layer with the fused random bias, and a bf16 layer again.  fp32 sums are added in a fixed order: same bits."""
    L = _lib.load()
    for case in ((64, 1000, 520, 16, 5, True, torch.float32, False),      # small k, one launch with tags
                 (24, 520, 1000, 16, 6, False, torch.float32, False),     # the same family, other layout of the array
                 (700, 264, 520, 136, 7, True, torch.float32, False),     # fp32 matrix cores
                 (300, 520, 264, 72, 8, False, torch.float32, True),      # ... with W = C.N + s.R
                 (512, 768, 512, 256, 9, True, torch.bfloat16, False)):
        print("case static scratch", case, flush=True)
        y, y_ref = _both(L, *case)
        assert torch.equal(y, y_ref) and bool(torch.isfinite(y.float()).all()), case


def test_static_scratch_rejects_what_does_not_fit():
    L = _lib.load()
    d = _desc(65536, 768, 3072, 256, 0)     # 64 MiB of projection state
    rc = L.rdb_linear_fwd_static(ctypes.c_void_p(256), 3072, ctypes.c_void_p(256), 768, ctypes.c_void_p(256), None, None, ctypes.byref(d), None)
    assert rc == -6 and b"static scratch holds" in L.rdb_last_error_string()
