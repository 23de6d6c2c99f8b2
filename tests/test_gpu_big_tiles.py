"""The 256-wide, persistent kernels of the projected entry points (k > 256) against the 128-wide ones and the CPU oracle.

Both kinds contract in the same order (stage after stage of 64, k-step after k-step of 16, fp32 accumulators of the same matrix
instruction), so y and dx must be equal bit for bit.  dcoef is equal bit for bit where the 128-wide kernels contract all tokens
in one range too (few tokens, or many output tiles); where they add up partial sums over token ranges the two differ by fp32
rounding only (1e-6 of the norm).  The oracle comparison holds the bf16 tolerance of the path (2e-2)."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

BF16_TOL = 2e-2


def rel_l2(a, b):
    a = np.asarray(a, dtype=np.float64)
    b = np.asarray(b, dtype=np.float64)
    return float(np.linalg.norm(a - b) / max(np.linalg.norm(b), 1e-30))


@pytest.fixture(scope="module")
def hip():
    assert torch.cuda.is_available(), "these tests need the MI355X"
    from randumb_amd import hip as h

    return h


def _inputs(T, in_f, out_f, k, seed):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(T, in_f, generator=g).bfloat16()
    dy = torch.randn(T, out_f, generator=g).bfloat16()
    coef = (torch.randn(out_f, k, generator=g) * (3.0 / k) ** 0.5 * 0.05).bfloat16()
    bias = torch.randn(out_f, generator=g).bfloat16()
    return x, dy, coef, bias


def _run(hip, mode, x, dy, coef, bias, in_f, out_f, k, seed, with_ct):
    before = hip.set_big_tiles(mode)
    try:
        z = hip.linear_project(x, k, out_f, seed, coef=coef if with_ct else None)
        y = hip.linear_fwd_projected(z, coef, in_f, seed, bias=bias)
        dx, dc = hip.linear_bwd_projected(dy, z, coef, in_f, seed)
        dc_alone = hip.linear_bwd_dcoef_projected(dy, z, k, in_f, seed)   # the coefficient gradient's own entry point
        torch.cuda.synchronize()
    finally:
        hip.set_big_tiles(before)
    # one pass over all tokens on the 256-wide tiles, fp32 atomics over token ranges on the 128-wide ones
    assert rel_l2(dc_alone.cpu().numpy(), dc.cpu().numpy()) < 1e-6
    if mode == 2:
        assert torch.equal(dc_alone, dc)
    return y, dx, dc


SHAPES = [
    # tokens, in_f, out_f, k, seed
    (300, 128, 264, 512, 2),      # one ragged tile in every direction
    (1000, 200, 520, 328, 5),     # k = 8 mod 16 (padded to 384 in the state), three output tiles, four token tiles
    (2088, 256, 4104, 1024, 7),   # many tiles: several rounds per block, a half-tile tail round, ragged edges
    (128, 64, 8, 264, 1),         # a single tile, mostly padding
]


@pytest.mark.parametrize("T,in_f,out_f,k,seed", SHAPES)
@pytest.mark.parametrize("with_ct", [True, False])
@pytest.mark.parametrize("with_bias", [True, False])
def test_big_tiles_equal_the_128_wide_kernels(hip, T, in_f, out_f, k, seed, with_ct, with_bias):
    print(f"case big tiles T={T} in={in_f} out={out_f} k={k} ct={with_ct} bias={with_bias}", flush=True)
    x, dy, coef, bias = [t.cuda() for t in _inputs(T, in_f, out_f, k, seed)]
    b = bias if with_bias else None
    want = _run(hip, 0, x, dy, coef, b, in_f, out_f, k, seed, with_ct)
    got = _run(hip, 2, x, dy, coef, b, in_f, out_f, k, seed, with_ct)
    for name, a, w in zip(("y", "dx"), got, want):
        assert a.shape == w.shape and torch.equal(a, w), f"{name} differs between the 256-wide and the 128-wide kernels"
    if T <= 256:   # a single token range in the 128-wide kernels as well
        assert torch.equal(got[2], want[2])
    assert got[2].shape == want[2].shape and rel_l2(got[2].cpu().numpy(), want[2].cpu().numpy()) < 1e-6
    # twice in a row on the same buffers: the same bits (no atomics, no state left behind by the persistent blocks)
    again = _run(hip, 2, x, dy, coef, b, in_f, out_f, k, seed, with_ct)
    for a, w in zip(again, got):
        assert torch.equal(a, w)


def test_big_tiles_against_the_oracle(hip, oracle):
    T, in_f, out_f, k, seed = 520, 136, 528, 384, 11
    print(f"case big tiles oracle T={T} in={in_f} out={out_f} k={k}", flush=True)
    x, dy, coef, bias = _inputs(T, in_f, out_f, k, seed)
    xn, dyn, cn = x.float().numpy(), dy.float().numpy(), coef.float().numpy()
    want_y = oracle.linear_fwd(xn, cn, in_f, out_f, seed, bias=bias.float().numpy())
    want_dx, want_dc, _ = oracle.linear_bwd(xn, dyn, cn, in_f, out_f, seed)
    y, dx, dc = _run(hip, 2, x.cuda(), dy.cuda(), coef.cuda(), bias.cuda(), in_f, out_f, k, seed, True)
    assert rel_l2(y.float().cpu().numpy(), want_y) < BF16_TOL
    assert rel_l2(dx.float().cpu().numpy(), want_dx) < BF16_TOL
    assert rel_l2(dc.float().cpu().numpy(), want_dc) < BF16_TOL


def test_big_tiles_run_by_default_on_a_layer_with_many_tiles(hip):
    """4096 -> 14336 with k = 1024 at 4096 tokens takes the 256-wide kernels without being asked to: same bits as with them off."""
    T, in_f, out_f, k, seed = 4096, 4096, 14336, 1024, 0
    print("case big tiles default", flush=True)
    x, dy, coef, _ = [t.cuda() for t in _inputs(T, in_f, out_f, k, seed)]
    assert hip.set_big_tiles(1) == 1   # the default mode
    got = _run(hip, 1, x, dy, coef, None, in_f, out_f, k, seed, True)
    want = _run(hip, 0, x, dy, coef, None, in_f, out_f, k, seed, True)
    for a, w in zip(got, want):
        assert torch.equal(a, w)


def test_big_tiles_random_shapes(hip):
    """Sixteen random layers with k > 256 (sizes in multiples of 8, tokens any number, ragged against every tile edge), with
    the transposed coefficients in the state or not, with the ordered-sum workspace or the smaller one."""
    rng = np.random.default_rng(31)
    for case in range(16):
        T = int(rng.integers(1, 160)) * 8 - int(rng.integers(0, 8))
        in_f, out_f = (int(rng.integers(1, 100)) * 8 for _ in range(2))
        k = int(rng.integers(33, 130)) * 8                      # 264 .. 1032
        seed = int(rng.integers(0, 2**32))
        print(f"case big tiles random {case}: T={T} in={in_f} out={out_f} k={k} seed={seed}", flush=True)
        x, dy, coef, bias = [t.cuda() for t in _inputs(T, in_f, out_f, k, case)]
        b = bias if case % 2 else None
        outs = {}
        for mode in (0, 2):
            before = hip.set_big_tiles(mode)
            try:
                z = hip.linear_project(x, k, out_f, seed, coef=coef if case % 3 else None)
                y = hip.linear_fwd_projected(z, coef, in_f, seed, bias=b)
                dx, dc = hip.linear_bwd_projected(dy, z, coef, in_f, seed, ordered_sums=case % 4 != 0)
                torch.cuda.synchronize()
            finally:
                hip.set_big_tiles(before)
            outs[mode] = (y, dx, dc)
        assert torch.equal(outs[2][0], outs[0][0]) and torch.equal(outs[2][1], outs[0][1]), case
        assert rel_l2(outs[2][2].cpu().numpy(), outs[0][2].cpu().numpy()) < 1e-5, case   # atomics / token ranges in the 128-wide kernels


def test_big_tiles_take_leading_dimensions(hip):
    """dy as a column slice of a wider matrix and y, dx written into wider matrices: same bits as on contiguous buffers."""
    import ctypes

    from randumb_amd import _lib
    from randumb_amd.hip import RDB_OP_LINEAR_BWD_PROJECTED, _p, _proj_desc, _stream

    print("case big tiles on strided activations", flush=True)
    T, in_f, out_f, k, seed = 700, 264, 520, 520, 4
    g = torch.Generator().manual_seed(8)
    x = torch.randn(T, in_f, generator=g).bfloat16().cuda()
    dyw = torch.randn(T, out_f + 24, generator=g).bfloat16().cuda()
    C = (torch.randn(out_f, k, generator=g) * 0.05).bfloat16().cuda()
    dy = dyw[:, 8:8 + out_f]
    L = _lib.load()
    before = hip.set_big_tiles(2)
    try:
        z = hip.linear_project(x, k, out_f, seed, coef=C)
        y_c = hip.linear_fwd_projected(z, C, in_f, seed)
        dx_c, dC_c = hip.linear_bwd_projected(dy.contiguous(), z, C, in_f, seed)
        d = _proj_desc(T, in_f, out_f, k, seed)
        yw = torch.full((T, out_f + 40), 7.0, dtype=torch.bfloat16, device="cuda")
        dxw = torch.full((T, in_f + 16), 7.0, dtype=torch.bfloat16, device="cuda")
        dC = torch.empty(out_f, k, dtype=torch.float32, device="cuda")
        y, dx = yw[:, 16:16 + out_f], dxw[:, 8:8 + in_f]
        n = L.rdb_linear_workspace_bytes(RDB_OP_LINEAR_BWD_PROJECTED, ctypes.byref(d))
        ws = torch.empty(max(n, 16), dtype=torch.uint8, device="cuda")
        st = _stream(x.device)
        _lib.check(L.rdb_linear_fwd_projected(_p(y), y.stride(0), _p(z), _p(C), None, ctypes.byref(d), st), "rdb_linear_fwd_projected")
        _lib.check(L.rdb_linear_bwd_projected(_p(dx), dx.stride(0), _p(dC), _p(dy), dy.stride(0), _p(z), _p(C), ctypes.byref(d), _p(ws), n, st),
                   "rdb_linear_bwd_projected")
        torch.cuda.synchronize()
    finally:
        hip.set_big_tiles(before)
    assert torch.equal(y, y_c) and torch.equal(dx, dx_c) and torch.equal(dC, dC_c)
    # nothing outside the slices was written
    assert bool((yw[:, :16] == 7).all()) and bool((yw[:, 16 + out_f:] == 7).all())
    assert bool((dxw[:, :8] == 7).all()) and bool((dxw[:, 8 + in_f:] == 7).all())


def test_big_tiles_through_the_layer(hip):
    """SillyLinear in matrix-coef form with k = 512: forward, backward and the gradients of input and coefficients are the
    same with the 256-wide kernels as with the 128-wide ones (autograd function, custom ops and C ABI in between)."""
    import randumb_amd as rten

    print("case big tiles through SillyLinear", flush=True)
    torch.manual_seed(3)
    outs = {}
    for mode in (0, 2):
        before = hip.set_big_tiles(mode)
        try:
            assert hip.linear_projection_preferred(300, 1032, 2056, 512)   # the projected kernels are what the layer runs
            layer = rten.SillyLinear(1032, 2056, [512, 512], [9, 10], bias=False, matrix_coef=True).to(torch.bfloat16).cuda()
            with torch.no_grad():
                g = torch.Generator().manual_seed(5)
                layer.weight_coef.copy_((torch.randn(2056, 512, generator=g) * 0.02).bfloat16())
                layer.weight_scale_bias.zero_()
            x = torch.randn(300, 1032, generator=torch.Generator().manual_seed(6)).bfloat16().cuda().requires_grad_(True)
            y = layer(x)
            (y.float() ** 2).sum().backward()
            torch.cuda.synchronize()
            outs[mode] = (y.detach(), x.grad.detach(), layer.weight_coef.grad.detach())
        finally:
            hip.set_big_tiles(before)
    assert torch.equal(outs[2][0], outs[0][0]) and torch.equal(outs[2][1], outs[0][1])
    assert rel_l2(outs[2][2].float().cpu().numpy(), outs[0][2].float().cpu().numpy()) < 1e-2   # bf16 gradients of fp32 sums in two orders
    assert float(outs[2][2].float().abs().sum()) > 0


def test_big_tiles_on_chunked_tokens(hip):
    """40000 tokens x 14336 output features hold more elements than one launch addresses: the projected calls run the layer
    in chunks of tokens, the later chunks adding to dcoef.  Same y and dx bit for bit on both kinds of kernels, same dcoef up to
    the order of fp32 sums, and the same dcoef bit for bit on a second run."""
    T, in_f, out_f, k, seed = 40000, 256, 14336, 512, 3
    print(f"case big tiles chunked T={T} in={in_f} out={out_f} k={k}", flush=True)
    g = torch.Generator().manual_seed(12)
    x = torch.randn(T, in_f, generator=g).bfloat16().cuda()
    dy = (torch.randn(T, 64, generator=g).bfloat16().cuda()).repeat(1, out_f // 64)   # cheap to make, still different per column block
    dy = dy * torch.linspace(0.5, 1.5, out_f, device="cuda").bfloat16()
    coef = (torch.randn(out_f, k, generator=g) * 0.01).bfloat16().cuda()
    outs = {}
    for mode in (0, 2, 2):
        before = hip.set_big_tiles(mode)
        try:
            z = hip.linear_project(x, k, out_f, seed, coef=coef)
            y = hip.linear_fwd_projected(z, coef, in_f, seed)
            dx, dc = hip.linear_bwd_projected(dy, z, coef, in_f, seed)
            torch.cuda.synchronize()
        finally:
            hip.set_big_tiles(before)
        if mode in outs:   # second run on the 256-wide kernels
            assert torch.equal(outs[mode][2], dc) and torch.equal(outs[mode][0], y)
        outs[mode] = (y, dx, dc)
        del z
    assert torch.equal(outs[2][0], outs[0][0]) and torch.equal(outs[2][1], outs[0][1])
    assert rel_l2(outs[2][2].cpu().numpy(), outs[0][2].cpu().numpy()) < 1e-5
    assert float(outs[2][2].abs().sum()) > 0
