"""Host-side behaviour of the Python surface that needs no GPU: lazy view ops, constructor contract, layer
parameter/buffer names, init formulas, seed generators, C-ABI symbol table.  Written from the reference's source
text (src/rten_cpp/RandumbTensor.py:794-994, src/rten_cpp/SillyLayers.py)."""
import ctypes
import math
import os
import re

import pytest
import torch

import randumb_amd as ra
from randumb_amd import CreateRandumbTensor, RandumbTensor, SillyConv2d, SillyLinear, listgen, stepgen

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_library_exports_every_declared_symbol():
    """The shared library loads without a GPU and exports exactly what include/randumb_hip.h declares."""
    from randumb_amd import _lib

    hdr = open(os.path.join(ROOT, "include", "randumb_hip.h")).read()
    declared = set(re.findall(r"\b(rdb_[a-z0-9_]+)\s*\(", hdr))
    assert declared == set(_lib.EXPORTS), declared ^ set(_lib.EXPORTS)
    lib = ctypes.CDLL(_lib.SO_PATH)
    for name in declared:
        assert hasattr(lib, name), name
    assert _lib.load().rdb_abi_version() == _lib.ABI_VERSION == 8
    assert ctypes.sizeof(_lib.LinearDesc) == 7 * 8 + 4 * 4


def test_loader_refuses_a_library_of_another_abi_version(monkeypatch):
    """A library that exports the same names with another ABI version is refused at load, not called with shifted arguments."""
    from randumb_amd import _lib

    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "ABI_VERSION", 7)
    with pytest.raises(_lib.RandumbHipError, match="ABI version 8"):
        _lib.load()
    monkeypatch.setattr(_lib, "ABI_VERSION", 8)
    assert _lib.load().rdb_abi_version() == 8


def test_one_launch_switch_without_a_gpu():
    """rdb_set_one_launch returns the previous mode and starts at 1; the counter queries refuse a NULL destination."""
    from randumb_amd import _lib

    L = _lib.load()
    assert L.rdb_set_one_launch(0) == 1 and L.rdb_set_one_launch(5) == 0 and L.rdb_set_one_launch(1) == 1
    assert L.rdb_sync_giveups_async(None, None) == -1 and L.rdb_sync_giveups(None, None) == -1


def test_sync_watch_host_logic():
    """The host side of the one-launch kernels' bounded waits, with the library and the device stubbed out: the counter is
    copied every `every` calls, looked at only when the copy has arrived, and a change switches the library to separate
    launches and raises once (a later unchanged counter does not raise again)."""
    from randumb_amd import _lib, hip

    class FakeEvent:
        done = False

        def record(self):
            pass

        def query(self):
            return self.done

        def synchronize(self):
            self.done = True

    class FakeLib:
        counter = 0
        one_launch = 1
        copies = 0

        def __init__(self, host):
            self.host = host

        def rdb_sync_giveups_async(self, dst, stream):
            self.copies += 1
            self.host[0] = self.counter
            return 0

        def rdb_set_one_launch(self, mode):
            old, self.one_launch = self.one_launch, mode
            return old

    host = torch.zeros(1, dtype=torch.int32)
    lib = FakeLib(host)
    events = []

    def make_event():
        events.append(FakeEvent())
        return events[-1]

    w = hip.SyncWatch(lib=lib, host_word=host, event_factory=make_event, every=4)
    for _ in range(3):
        w.tick(None)
    assert lib.copies == 0 and w.pending is None
    w.tick(None)                      # 4th call: a copy is enqueued, nothing is waited for
    assert lib.copies == 1 and w.pending is events[0]
    for _ in range(10):
        w.tick(None)                  # the copy has not arrived: no look, no second copy
    assert lib.copies == 1 and lib.one_launch == 1
    events[0].done = True
    w.tick(None)                      # arrived, counter unchanged: fine
    assert w.pending is None and lib.one_launch == 1
    lib.counter = 3                   # three blocks give up
    w.tick(None)                      # call 16: next copy
    assert lib.copies == 2
    events[1].done = True
    with pytest.raises(_lib.RandumbHipError, match="3 block"):
        w.tick(None)
    assert lib.one_launch == 0 and w.seen == 3
    w.check(None)                     # an explicit look waits for the copy; the counter has not moved since: no error
    lib.counter = 4
    with pytest.raises(_lib.RandumbHipError, match="1 block"):
        w.check(None)


def test_big_tiles_switch_without_a_gpu():
    """rdb_set_big_tiles returns the previous mode, clamps to 0..2 and starts at 1 (the 256-wide kernels by the tile-count rule)."""
    from randumb_amd import _lib

    L = _lib.load()
    first = L.rdb_set_big_tiles(0)
    try:
        assert first == 1
        assert L.rdb_set_big_tiles(7) == 0 and L.rdb_set_big_tiles(-3) == 2 and L.rdb_set_big_tiles(2) == 0
    finally:
        L.rdb_set_big_tiles(first)
    assert L.rdb_set_big_tiles(first) == first


def test_f32_split_switch_without_a_gpu():
    """rdb_set_f32_split returns the previous mode and starts at 1 (fp32 products as three-way bf16 splits)."""
    from randumb_amd import _lib

    L = _lib.load()
    first = L.rdb_set_f32_split(0)
    try:
        assert first == 1
        assert L.rdb_set_f32_split(5) == 0 and L.rdb_set_f32_split(0) == 1
    finally:
        L.rdb_set_f32_split(first)
    assert L.rdb_set_f32_split(first) == first


def test_argument_errors_come_back_as_codes_without_a_gpu():
    from randumb_amd import _lib

    L = _lib.load()
    assert L.rdb_sq5_fill_2d(None, -1, 4, 0, None) == -2
    assert b"negative" in L.rdb_last_error_string()
    assert L.rdb_sq5_fill_2d(None, 4, 4, 0, None) == -1
    assert L.rdb_sq5_fill_2d(None, 0, 4, 0, None) == 0  # empty: nothing to do, no pointer needed
    assert L.rdb_materialize_fwd(None, None, 7, 0, 4, 0, 2, 2, 2, 1, 0, None, None) == -3
    d = _lib.LinearDesc()
    d.tokens, d.in_f, d.out_f, d.k, d.coef_rows, d.sO, d.sI = 4, 8, 6, 3, 5, 8, 1
    assert L.rdb_linear_fwd(None, 6, None, 8, None, None, None, ctypes.byref(d), None, 0, None) == -2  # coef_rows != out_f
    assert L.rdb_linear_fwd(None, 6, None, 8, None, None, None, None, None, 0, None) == -1
    assert L.rdb_materialize_bwd_workspace_bytes(0, 256, 0, 2359296) > 0
    # matrix-coef, large enough for the matrix-core kernels: one [rows x k] matrix per range of the row (here 768 / 256 = 3)
    assert L.rdb_materialize_bwd_workspace_bytes(3072, 256, 768, 2359296) == 3 * 3072 * 256 * 4
    assert L.rdb_materialize_bwd_workspace_bytes(10, 64, 256, 2560) == 0


def test_workspace_queries_and_projected_argument_checks_without_a_gpu():
    """Host logic of the fused-linear entry points: scratch sizes, which layers qualify for the projected form, and argument
    errors that must come back before anything touches a GPU."""
    from randumb_amd import _lib

    L = _lib.load()

    def desc(tokens, in_f, out_f, k, act=_lib.RDB_BF16, coef=_lib.RDB_BF16, rows=None, algo=_lib.RDB_ALGO_AUTO):
        d = _lib.LinearDesc()
        d.tokens, d.in_f, d.out_f, d.k, d.coef_rows, d.sO, d.sI = tokens, in_f, out_f, k, out_f if rows is None else rows, in_f, 1
        d.act_dtype, d.coef_dtype, d.algo = act, coef, algo
        return d

    d = desc(8192, 768, 3072, 256)
    r = ctypes.byref(d)
    zbytes = 8192 * 256 * 2

    def state_bytes(tokens, in_f, out_f, k):
        # header + z for the forward product (tokens to 32) + z transposed (tokens to 64) + C transposed (out to 64)
        # + per 256 tokens a 64-bit slot per projection tile (32 coefficients) and one counter
        up = lambda n, m: -(-n // m) * m
        kpad = up(k, 64)
        zf = up(tokens, 32) * kpad * 2
        return (256 + up(zf, 256) + up(up(tokens, 64) * kpad * 2, 256) + up(up(out_f, 64) * kpad * 2, 256)
                + up(-(-tokens // 256) * (kpad // 32 + 1) * 8, 256))

    assert state_bytes(8192, 768, 3072, 256) == 256 + 2 * zbytes + 3072 * 256 * 2 + 32 * 9 * 8
    assert L.rdb_linear_projection_bytes(r) == state_bytes(8192, 768, 3072, 256)
    info = (ctypes.c_int64 * 8)()
    assert L.rdb_linear_projection_layout(r, info) == 0
    assert list(info) == [256, 1, 256 + zbytes, 256 + 2 * zbytes, 256, 8192, 8192, 3072]
    assert L.rdb_linear_projection_bytes(ctypes.byref(desc(1000, 200, 328, 72))) == state_bytes(1000, 200, 328, 72)
    assert L.rdb_linear_projection_bytes(ctypes.byref(desc(4096, 4096, 14336, 1024))) == state_bytes(4096, 4096, 14336, 1024)
    assert L.rdb_linear_workspace_bytes(_lib.RDB_OP_LINEAR_FWD, r) == state_bytes(8192, 768, 3072, 256)
    assert L.rdb_linear_workspace_bytes(_lib.RDB_OP_LINEAR_BWD_DX, r) == zbytes
    assert L.rdb_linear_workspace_bytes(_lib.RDB_OP_LINEAR_BWD_DCOEF, r) == state_bytes(8192, 768, 3072, 256)
    # whole backward pass: dy.C plus the partial sums of the coefficient gradient, one [out x k] fp32 matrix per token split
    extra = L.rdb_linear_workspace_bytes(_lib.RDB_OP_LINEAR_BWD_PROJECTED, r) - zbytes
    assert extra > 0 and extra % (3072 * 256 * 4) == 0
    # dy.C is kept padded (tokens to 32, k to 64) for the kernel that holds it in registers, unless that would pass the
    # operand size limit: then it stays [tokens x k]
    assert L.rdb_linear_workspace_bytes(_lib.RDB_OP_LINEAR_BWD_DX, ctypes.byref(desc(1000, 200, 328, 72))) == 1024 * 128 * 2
    assert L.rdb_linear_workspace_bytes(_lib.RDB_OP_LINEAR_BWD_DX, ctypes.byref(desc((1 << 26) - 8, 768, 3072, 8))) == ((1 << 26) - 8) * 8 * 2
    # the random-bias share on its own: one float per tile of 64 features x 256 tokens for the scale's gradient; argument checks
    assert L.rdb_linear_workspace_bytes(_lib.RDB_OP_LINEAR_RBIAS_BWD, r) == (768 // 64) * (8192 // 256) * 4
    assert L.rdb_linear_workspace_bytes(_lib.RDB_OP_LINEAR_RBIAS_BWD, ctypes.byref(desc(8192, 768, 3072, 256, act=_lib.RDB_F32, coef=_lib.RDB_F32))) == 0
    assert L.rdb_linear_rbias_fwd(None, 3072, None, 768, None, r, None) == -1
    fake = ctypes.c_void_p(256)   # never dereferenced: the calls below are refused before any launch
    assert L.rdb_linear_rbias_fwd(fake, 3071, fake, 768, fake, r, None) == -2
    assert L.rdb_linear_rbias_fwd(fake, 3072, fake, 768, fake, ctypes.byref(desc(8192, 768, 3072, 256, act=_lib.RDB_F32, coef=_lib.RDB_F32)), None) == -5
    assert L.rdb_linear_rbias_bwd(fake, 776, None, fake, 3072, None, 0, fake, ctypes.byref(desc(8192, 772, 3072, 256)), None, 0, None) == -5
    ds = ctypes.c_void_p(512)
    assert L.rdb_linear_rbias_bwd(fake, 768, ds, fake, 3072, None, 0, fake, r, None, 0, None) == -1          # d s needs x
    assert L.rdb_linear_rbias_bwd(fake, 768, ds, fake, 3072, fake, 768, fake, r, None, 0, None) == -6    # ... and scratch
    # kernels that form W tiles need no scratch; neither does a layer the factored form does not apply to
    for algo in (_lib.RDB_ALGO_TILE, _lib.RDB_ALGO_STRIP):
        assert L.rdb_linear_workspace_bytes(_lib.RDB_OP_LINEAR_FWD, ctypes.byref(desc(8192, 768, 3072, 256, algo=algo))) == 0
    assert L.rdb_linear_projection_bytes(ctypes.byref(desc(64, 100, 32, 16))) == 0                     # in_f % 8
    assert L.rdb_linear_projection_bytes(ctypes.byref(desc(64, 96, 32, 16, rows=0))) == 0              # vector-coef
    assert L.rdb_linear_projection_bytes(ctypes.byref(desc(64, 96, 32, 16, act=_lib.RDB_F32))) == 0    # fp32 activations
    assert L.rdb_linear_projection_bytes(None) == 0
    # activations of 2^29 elements or more are outside one launch's 32-bit addressing: the layer is run in chunks of tokens,
    # each with a state of its own (chunks of at most 2^28 / widest row tokens, a multiple of 256, about equal)
    ct = ctypes.c_int64()
    assert L.rdb_linear_projection_chunks(r, ctypes.byref(ct)) == 1 and ct.value == 8192
    big = desc(65536, 4096, 14336, 256)
    assert L.rdb_linear_projection_chunks(ctypes.byref(big), ctypes.byref(ct)) == 4 and ct.value == 16384   # 2^28 / 14336 = 18724 -> 18688
    assert L.rdb_linear_projection_bytes(ctypes.byref(big)) == 4 * state_bytes(16384, 4096, 14336, 256)
    odd = desc(40000, 4096, 14336, 256)                                                   # 3 chunks of 13568, 13568, 12864
    assert L.rdb_linear_projection_chunks(ctypes.byref(odd), ctypes.byref(ct)) == 3 and ct.value == 13568
    assert L.rdb_linear_projection_bytes(ctypes.byref(odd)) == 3 * state_bytes(13568, 4096, 14336, 256)
    assert L.rdb_linear_projection_chunks(ctypes.byref(desc(1 << 21, 768, 3072, 256)), ctypes.byref(ct)) == 25 and ct.value % 256 == 0
    assert ct.value * 3072 < (1 << 28) + 256 * 3072
    # chunks after the first add to dcoef: their sums pass through the workspace even when a chunk is a single token range
    w_big = L.rdb_linear_workspace_bytes(_lib.RDB_OP_LINEAR_BWD_PROJECTED, ctypes.byref(big))
    w_one = L.rdb_linear_workspace_bytes(_lib.RDB_OP_LINEAR_BWD_PROJECTED, ctypes.byref(desc(16384, 4096, 14336, 256)))
    assert w_big >= w_one >= 16384 * 256 * 2 and (w_big - 16384 * 256 * 2) % (14336 * 256 * 4) == 0
    assert L.rdb_linear_projection_layout(ctypes.byref(big), info) == -5 and b"4 states" in L.rdb_last_error_string()
    # fp32, small k: one partial [tokens x k] matrix per 256 values of the longer side, a 64-bit tag slot per tile of 8 tokens
    # and chunk, a word for a block that gave up waiting, and a counter per 16 tokens
    # ... or, for the fp32 matrix-core kernels (any k, sizes that are multiples of 4), z [tokens x k] rounded up to 256 bytes plus
    # one partial matrix per range of the contraction when the [tokens x k] product has fewer tiles than two per compute unit
    # (256 units without a GPU; ranges of at least 128 values, at most 32): here one tile, 4096 / 128 = 32 ranges.  The query
    # returns the larger of the two.
    f32 = desc(16, 4096, 4096, 16, act=_lib.RDB_F32, coef=_lib.RDB_F32)
    small_k = 16 * 16 * 16 * 4 + 2 * 16 * 8 + 8 + 8
    assert L.rdb_linear_workspace_bytes(_lib.RDB_OP_LINEAR_FWD, ctypes.byref(f32)) == max(small_k, 1024 * (1 + 32))
    k128 = desc(16, 4096, 4096, 128, act=_lib.RDB_F32, coef=_lib.RDB_F32)
    assert L.rdb_linear_workspace_bytes(_lib.RDB_OP_LINEAR_FWD, ctypes.byref(k128)) == 16 * 128 * 4 * (1 + 32)
    # bf16 with a few tokens (up to 96, k up to 256): the vector-ALU kernels' scratch where it is the larger need (16 chunks of
    # 256 features, a [16 x 256] fp32 matrix each, and their sum): for the input gradient, whose matrix-core form
    # needs only t; the other two calls' need stays the projection state's.  Beyond 96 tokens the few-token kernels are out.
    few16 = 16 * 16 * 256 * 4 + 16 * 256 * 4   # the chunks' partial matrices and their sum
    assert L.rdb_linear_workspace_bytes(_lib.RDB_OP_LINEAR_BWD_DX, ctypes.byref(desc(16, 4096, 4096, 256))) == few16
    assert L.rdb_linear_workspace_bytes(_lib.RDB_OP_LINEAR_BWD_DX, ctypes.byref(desc(97, 4096, 4096, 256))) == 128 * 256 * 2
    for op in (_lib.RDB_OP_LINEAR_FWD, _lib.RDB_OP_LINEAR_BWD_DCOEF):
        assert L.rdb_linear_workspace_bytes(op, ctypes.byref(desc(16, 4096, 4096, 256))) == state_bytes(16, 4096, 4096, 256) > few16
    assert L.rdb_linear_workspace_bytes(_lib.RDB_OP_LINEAR_FWD, ctypes.byref(desc(97, 4096, 4096, 256))) == state_bytes(97, 4096, 4096, 256)
    # 8192 tokens x 256 coefficients are 128 tiles of 128 x 128: four ranges; the coefficient gradient's 48 tiles: ten ranges of
    # tokens, one [out_f x k] matrix each
    c2 = desc(8192, 768, 3072, 256, act=_lib.RDB_F32, coef=_lib.RDB_F32)
    assert L.rdb_linear_workspace_bytes(_lib.RDB_OP_LINEAR_FWD, ctypes.byref(c2)) == 8192 * 256 * 4 * (1 + 4)
    assert L.rdb_linear_workspace_bytes(_lib.RDB_OP_LINEAR_BWD_DX, ctypes.byref(c2)) == 8192 * 256 * 4 * (1 + 4)
    # ... and a value per 64 x 128 tile of [tokens x out_f] for the gradient of the random bias's scale
    assert L.rdb_linear_workspace_bytes(_lib.RDB_OP_LINEAR_BWD_DCOEF, ctypes.byref(c2)) == 8192 * 256 * 4 * (1 + 4) + 10 * 3072 * 256 * 4 + 128 * 24 * 4
    # enough tiles: no ranges
    wide = desc(65536, 768, 3072, 256, act=_lib.RDB_F32, coef=_lib.RDB_F32)
    assert L.rdb_linear_workspace_bytes(_lib.RDB_OP_LINEAR_FWD, ctypes.byref(wide)) == 65536 * 256 * 4
    # extents that are not multiples of 4 run on the same kernels (operands read value by value): same scratch
    assert L.rdb_linear_workspace_bytes(_lib.RDB_OP_LINEAR_FWD, ctypes.byref(desc(16, 4096, 4094, 128, act=_lib.RDB_F32, coef=_lib.RDB_F32))) == 16 * 128 * 4 * (1 + 32)
    # bf16 sizes that are not multiples of 8 run on these kernels too (bf16 read value by value, z and t kept in fp32)
    odd16 = desc(16, 4096, 4094, 128)
    assert L.rdb_linear_workspace_bytes(_lib.RDB_OP_LINEAR_FWD, ctypes.byref(odd16)) == 16 * 128 * 4 * (1 + 32)
    # vector-coef, up to 4096 tokens: one fp32 partial output per 32 values of the contraction; beyond: the general kernel, no scratch
    vec = desc(16, 4096, 4096, 128, rows=0, act=_lib.RDB_F32, coef=_lib.RDB_F32)
    assert L.rdb_linear_workspace_bytes(_lib.RDB_OP_LINEAR_FWD, ctypes.byref(vec)) == (4096 // 32) * 16 * 4096 * 4
    assert L.rdb_linear_workspace_bytes(_lib.RDB_OP_LINEAR_BWD_DX, ctypes.byref(vec)) == (4096 // 32) * 16 * 4096 * 4
    # its coefficient gradient: room for dW = dy^T.x (fp32; here one range of tokens) and for what contracting it needs
    up256 = lambda n: -(-n // 256) * 256
    L.rdb_materialize_bwd_workspace_bytes.restype = ctypes.c_int64
    L.rdb_scale_bias_bwd_workspace_bytes.restype = ctypes.c_int64
    nw = 4096 * 4096
    want = nw * 4 + up256(L.rdb_materialize_bwd_workspace_bytes(ctypes.c_int64(0), ctypes.c_int64(128), ctypes.c_int64(0), ctypes.c_int64(nw))) \
        + up256(L.rdb_scale_bias_bwd_workspace_bytes(ctypes.c_int64(nw)))
    assert L.rdb_linear_workspace_bytes(_lib.RDB_OP_LINEAR_BWD_DCOEF, ctypes.byref(vec)) == want
    # ... only for a weight that is contiguous in memory
    tr = desc(16, 4096, 4096, 128, rows=0, act=_lib.RDB_F32, coef=_lib.RDB_F32)
    tr.sO, tr.sI = 1, 4096
    assert L.rdb_linear_workspace_bytes(_lib.RDB_OP_LINEAR_BWD_DCOEF, ctypes.byref(tr)) == 0
    assert L.rdb_linear_workspace_bytes(_lib.RDB_OP_LINEAR_FWD, ctypes.byref(desc(8192, 4096, 4096, 128, rows=0, act=_lib.RDB_F32, coef=_lib.RDB_F32))) == 0

    bad = ctypes.byref(desc(64, 100, 32, 16))
    assert L.rdb_linear_project(None, None, 100, None, bad, None) == -5  # RDB_E_UNSUPPORTED
    assert b"projected form" in L.rdb_last_error_string()
    assert L.rdb_linear_project(None, None, 768, None, r, None) == -1                                    # NULL pointers
    assert L.rdb_linear_fwd_projected(None, 3072, None, None, None, r, None) == -1
    assert L.rdb_linear_bwd_dcoef_projected(None, None, 3072, None, r, None) == -1
    assert L.rdb_linear_bwd_projected(None, 768, None, None, 3072, None, None, r, None, 0, None) == -1
    assert L.rdb_linear_fwd_projected(ctypes.c_void_p(16), 8, ctypes.c_void_p(16), ctypes.c_void_p(16), None, r, None) == -2  # ldy < out_f
    assert L.rdb_linear_project(None, None, 768, None, None, None) == -1
    assert L.rdb_linear_project_fwd(None, 3072, None, None, 768, None, None, r, None) == -1                 # NULL pointers
    p16 = ctypes.c_void_p(16)
    assert L.rdb_linear_project_fwd(p16, 8, p16, p16, 768, p16, None, r, None) == -2                        # ldy < out_f
    assert L.rdb_linear_project_fwd(p16, 3072, p16, p16, 8, p16, None, r, None) == -2                       # ldx < in_f
    assert L.rdb_linear_project_fwd(p16, 3072, p16, ctypes.c_void_p(24), 768, p16, None, r, None) == -5     # x not 16-byte aligned
    assert L.rdb_linear_project_fwd(None, 32, None, None, 100, None, None, bad, None) == -5                 # the form does not apply


def test_view_ops_stay_lazy_and_only_change_shape_and_stride():
    c = torch.nn.Parameter(torch.randn(18))
    rt = CreateRandumbTensor(c, 1337, (3, 6))
    assert isinstance(rt, RandumbTensor) and rt.shape == (3, 6) and rt.stride() == (6, 1)
    assert rt.int_dim == 18 and rt.noise_matrix_shape == (18, 18) and rt.seed == 1337 and rt._coef is c
    t = rt.t()
    assert isinstance(t, RandumbTensor) and t.shape == (6, 3) and t.stride() == (1, 6) and t._coef is c
    assert rt.transpose(0, 1).stride() == (1, 6)
    assert rt.view(6, 3).stride() == (3, 1)
    assert rt.view(2, 3, 3).permute(2, 0, 1).shape == (3, 2, 3)
    assert rt.permute(1, 0).stride() == (1, 6)
    with pytest.raises(RuntimeError, match="view size is not compatible"):
        rt.t().view(18)
    b = rt.to(torch.bfloat16)
    assert isinstance(b, RandumbTensor) and b.dtype == torch.bfloat16 and b._coef is c
    assert rt._tensor is None


def test_constructor_contract():
    c = torch.nn.Parameter(torch.randn(5))
    rt = CreateRandumbTensor(c, 3, (4, 2))
    assert rt.requires_grad and rt.grad_fn is not None and rt.dtype == c.dtype and rt.device == c.device
    with pytest.raises(AssertionError):
        CreateRandumbTensor(torch.randn(2, 3, 4), 0, (4, 2))
    with pytest.raises(AssertionError):  # matrix-coef needs (rows, row_len)
        CreateRandumbTensor(torch.randn(3, 4), 0, (4, 2))
    m = CreateRandumbTensor(torch.randn(4, 7), 0, (4, 9))
    assert m.coef_rows == 4 and m.row_len == 9 and m.noise_matrix_shape == (9, 7)
    assert m.t().row_len == 9
    with pytest.raises(NotImplementedError):  # no CPU implementation, as in the reference
        rt + 1


def test_seed_generators():
    g = stepgen(10, 3)
    assert [next(g) for _ in range(4)] == [10, 13, 16, 19]
    assert list(listgen([5, 7, 9])) == [5, 7, 9]


def test_silly_linear_surface():
    ints, seeds = stepgen(64, 0), stepgen(1337, 1)
    l1 = SillyLinear(784, 256, ints, seeds)
    l2 = SillyLinear(256, 10, ints, seeds, bias=False)
    assert l1.seed == [1337, 1338] and l2.seed == [1339, 1340] and l1.int_dim == [64, 64]  # two draws per layer, bias or not
    assert sorted(n for n, _ in l1.named_parameters()) == ["bias_coef", "bias_scale_bias", "weight_coef", "weight_scale_bias"]
    assert sorted(n for n, _ in l1.named_buffers()) == ["bias", "weight"]
    assert sorted(l1.state_dict().keys()) == ["bias", "bias_coef", "bias_scale_bias", "weight", "weight_coef", "weight_scale_bias"]
    assert l2.bias is None and sorted(n for n, _ in l2.named_parameters()) == ["weight_coef", "weight_scale_bias"]
    assert l1.weight.shape == (256, 784) and l1.bias.shape == (256,) and l1.weight_coef.shape == (64,)
    # default init: zero coefficients, scale_bias = sqrt(3) * gain / sqrt(fan_in), gain = sqrt(2 / (1 + 5)) (SillyLayers.py:122-133)
    assert not l1.weight_coef.any() and not l1.bias_coef.any()
    want = math.sqrt(3.0) * math.sqrt(1.0 / 3.0) / math.sqrt(784)
    assert abs(float(l1.weight_scale_bias) - want) < 1e-7 and abs(float(l1.bias_scale_bias) - want) < 1e-7
    assert l1.weight.scale_bias is l1.weight_scale_bias and l1.weight._coef is l1.weight_coef
    m = SillyLinear(12, 5, [8, 8], [1, 2], matrix_coef=True)
    assert m.weight_coef.shape == (5, 8) and m.fused and m.weight.coef_rows == 5


def test_silly_conv2d_surface():
    """Constructor, parameter and buffer names, shapes and default init of the convolution layer (SillyLayers.py:230-297)."""
    ints, seeds = stepgen(64, 0), stepgen(1337, 1)
    c1 = SillyConv2d(1, 32, int_dim=ints, seed=seeds, kernel_size=3, stride=1, rt_bias=True)
    c2 = SillyConv2d(32, 64, int_dim=ints, seed=seeds, kernel_size=3, stride=1, rt_bias=True, bias=False)
    assert c1.seed == [1337, 1338] and c2.seed == [1339, 1340] and c1.int_dim == [64, 64]
    assert sorted(n for n, _ in c1.named_parameters()) == ["bias_coef", "bias_scale_bias", "weight_coef", "weight_scale_bias"]
    assert sorted(n for n, _ in c1.named_buffers()) == ["bias", "weight"]
    assert isinstance(c1.weight, RandumbTensor) and c1.weight.shape == (32, 1, 3, 3) and c1.weight.stride() == (9, 9, 3, 1)
    assert c1.bias.shape == (32,) and c1.weight_coef.shape == (64,) and c1.weight.fused_bias
    assert c2.bias is None and c2.weight.shape == (64, 32, 3, 3) and c2.weight.noise_matrix_shape == (64 * 32 * 9, 64)
    # default init: zero coefficients, scale_bias = sqrt(3) * gain / sqrt(fan_in) with fan_in = in_channels * kh * kw
    assert not c2.weight_coef.any()
    want = math.sqrt(3.0) * math.sqrt(1.0 / 3.0) / math.sqrt(32 * 9)
    assert abs(float(c2.weight_scale_bias) - want) < 1e-7
    c2 = c2.to(torch.bfloat16)
    assert c2.weight.dtype == torch.bfloat16 and c2.weight._coef is c2.weight_coef and c2.weight.shape == (64, 32, 3, 3)
    assert "int_dim=[64, 64]" in repr(c2)


def test_apply_rebuilds_tensors_on_the_converted_parameters():
    l = SillyLinear(12, 5, [8, 8], [1, 2])
    l = l.to(torch.bfloat16)
    assert l.weight.dtype == torch.bfloat16 and l.weight._coef is l.weight_coef and l.weight.scale_bias is l.weight_scale_bias
    assert l.bias._coef is l.bias_coef and isinstance(l.weight, RandumbTensor) and l.weight.requires_grad
    l = l.float()
    assert l.weight.dtype == torch.float32 and l.weight._coef is l.weight_coef


def test_init_variance_scaling():
    """var(coef) = 3 * std^2 / k  (uniform bound = 3 * std / sqrt(k)); bias uses the weight's fan-in and its own k."""
    l = SillyLinear(300, 50, [4096, 1024], [7, 8])
    ra.init_kaiming_uniform(l.weight, l.bias, 7)
    out_std = math.sqrt(1.0 / 3.0) / math.sqrt(300)
    for coef, k in ((l.weight_coef, 4096), (l.bias_coef, 1024)):
        bound = 3.0 * out_std / math.sqrt(k)
        assert float(coef.abs().max()) <= bound and float(coef.abs().max()) > 0.97 * bound
        assert abs(float(coef.var()) / (3 * out_std**2 / k) - 1) < 0.1
    l2 = SillyLinear(300, 50, [4096, 1024], [7, 8])
    ra.init_kaiming_uniform(l2.weight, l2.bias, 7)
    assert torch.equal(l.weight_coef, l2.weight_coef)  # seeded generator: reproducible
    m = SillyLinear(768, 64, [256, 256], [0, 1], matrix_coef=True, bias=False)
    ra.init_coef_normal(m.weight, 0.02, 0)
    assert abs(float(m.weight_coef.var()) / (3 * 0.02**2 / 256) - 1) < 0.05
    l.init_uniform_coef_zero_bias()
    assert float(l.weight_scale_bias) == 0.0 and l.weight_coef.any()


def test_materialised_weight_has_the_target_std(oracle):
    """README derivation: with var(coef) = 3 std^2 / k the weight entries have standard deviation std."""
    g = torch.Generator().manual_seed(0)
    k, std = 256, 0.02
    C = torch.randn(64, k, generator=g) * math.sqrt(3 * std**2 / k)
    W = oracle.materialize_fwd(C.numpy(), (64, 768), (768, 1), 5, row_len=768)
    assert abs(W.std() / std - 1) < 0.05
    c = torch.randn(k, generator=g) * math.sqrt(3 * std**2 / k)
    W1 = oracle.materialize_fwd(c.numpy(), (64, 768), (768, 1), 5)
    assert abs(W1.std() / std - 1) < 0.1


def test_projected_form_is_chosen_only_where_it_runs_and_pays():
    """ops.linear takes the projected form only for layers whose activations fit the kernels' addressing and for which the
    factored products are faster than forming the weight on chip; everything else goes to rten::linear_fwd (whose backward cannot
    be refused late, in the backward pass)."""
    from randumb_amd import hip

    assert hip.linear_projection_supported(8192, 768, 3072, 256) and hip.linear_projection_preferred(8192, 768, 3072, 256)
    # tokens*out_f >= 2^29 (65536 tokens x 14336): run in chunks of tokens by the library, so still the projected form
    assert hip.linear_projection_bytes(65536, 4096, 14336, 256) > 0
    assert hip.linear_projection_supported(65536, 4096, 14336, 256) and hip.linear_projection_preferred(65536, 4096, 14336, 256)
    assert hip.linear_projection_supported(1 << 17, 4096, 64, 8)
    # preferred up to k (in + out) = 16 in out: beyond the point where its flops equal those of a product on a stored weight
    # (768 -> 384 at k = 256), because the alternative is a kernel that forms the weight on chip
    assert hip.linear_projection_supported(512, 768, 384, 256) and hip.linear_projection_preferred(512, 768, 384, 256)
    assert hip.linear_projection_preferred(512, 768, 512, 256)
    assert hip.linear_projection_preferred(64, 64, 64, 64)        # ratio 2
    assert hip.linear_projection_supported(64, 8, 8, 64) and not hip.linear_projection_preferred(64, 8, 8, 64)   # ratio 16
    # ... and only while the state costs at most twice the memory of the x it is saved in place of: k (rounded up to 64) <= in_f
    assert hip.linear_projection_preferred(4096, 4096, 14336, 1024) and hip.linear_projection_preferred(300, 1032, 2056, 512)
    assert hip.linear_projection_supported(512, 256, 1024, 512) and not hip.linear_projection_preferred(512, 256, 1024, 512)
    assert not hip.linear_projection_preferred(64, 8, 8, 8)
    # the fused random bias has kernels of its own beside the projected calls in bf16 with sizes in multiples of 8 only
    import torch

    assert hip.linear_rbias_supported(768, 3072, torch.bfloat16) and not hip.linear_rbias_supported(768, 3072, torch.float32)
    assert not hip.linear_rbias_supported(772, 3072, torch.bfloat16) and not hip.linear_rbias_supported(768, 3076, torch.bfloat16)
