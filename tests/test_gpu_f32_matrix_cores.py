"""fp32 matrix-coef layers on the matrix cores (the factored algorithm, any k, many tokens) against the CPU oracle, at the
fp32 tolerance of the path (rel-L2 1e-5), and against the general kernel.  By default the products run as six bf16 matrix
instructions on exact three-way splits of the operands; test_split_products_are_as_accurate_as_fp32_instructions runs the fp32
matrix instructions beside them.

Asking for RDB_ALGO_FACTORED makes the library refuse rather than fall back to the general kernel, so a call that succeeds
with k > 64 (beyond the vector-ALU kernels for few tokens) ran these kernels."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

F32_TOL = 1e-5


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
    x = torch.randn(T, in_f, generator=g)
    dy = torch.randn(T, out_f, generator=g)
    coef = torch.randn(out_f, k, generator=g) * (3.0 / k) ** 0.5 * 0.05
    bias = torch.randn(out_f, generator=g)
    return x, dy, coef, bias


SHAPES = [
    # tokens, in_f, out_f, k, seed
    (512, 768, 1024, 128, 3),     # whole tiles
    (300, 260, 516, 68, 1337),    # ragged in every extent (multiples of 4)
    (64, 1024, 1024, 256, 5),     # few tokens: 64-row tiles
    (4500, 128, 256, 32, 9),      # small k, more tokens than the vector-ALU kernels take
    (4, 8, 12, 68, 1),            # smaller than one tile
    (2100, 516, 132, 100, 77),    # the coefficient gradient in several token ranges, ragged last range
    (333, 777, 555, 99, 8),       # no extent a multiple of 4: operands read value by value
    (130, 1001, 999, 102, 12),
    (7, 5, 3, 2, 3),
]


@pytest.mark.parametrize("T,in_f,out_f,k,seed", SHAPES)
def test_against_the_oracle(hip, oracle, T, in_f, out_f, k, seed):
    from randumb_amd._lib import RDB_ALGO_FACTORED

    print(f"case f32 matrix cores T={T} in={in_f} out={out_f} k={k}", flush=True)
    x, dy, coef, bias = _inputs(T, in_f, out_f, k, seed)
    xn, dyn, cn = x.numpy(), dy.numpy(), coef.numpy()
    want_y = oracle.linear_fwd(xn, cn, in_f, out_f, seed, bias=bias.numpy())
    want_dx, want_dc, _ = oracle.linear_bwd(xn, dyn, cn, in_f, out_f, seed)
    xc, dyc, cc = x.cuda(), dy.cuda(), coef.cuda()
    y = hip.linear_fwd(xc, cc, in_f, out_f, in_f, 1, seed, bias=bias.cuda(), algo=RDB_ALGO_FACTORED)
    assert y.dtype == torch.float32 and y.shape == (T, out_f)
    assert rel_l2(y.cpu().numpy(), want_y) < F32_TOL
    dx = hip.linear_bwd_dx(dyc, cc, in_f, out_f, in_f, 1, seed, algo=RDB_ALGO_FACTORED)
    assert rel_l2(dx.cpu().numpy(), want_dx) < F32_TOL
    dc, _ = hip.linear_bwd_dcoef(dyc, xc, k, out_f, in_f, out_f, in_f, 1, seed, algo=RDB_ALGO_FACTORED)
    assert dc.shape == coef.shape and rel_l2(dc.cpu().numpy(), want_dc) < F32_TOL
    # the same calls again give the same bits (token ranges are added in a fixed order)
    dc2, _ = hip.linear_bwd_dcoef(dyc, xc, k, out_f, in_f, out_f, in_f, 1, seed, algo=RDB_ALGO_FACTORED)
    assert torch.equal(dc, dc2)


def test_default_choice_and_the_general_kernel_agree(hip):
    """AUTO at a shape where the factored form is cheaper, against the kernel that forms W tiles (RDB_ALGO_TILE)."""
    from randumb_amd._lib import RDB_ALGO_TILE

    T, in_f, out_f, k, seed = 2048, 384, 640, 96, 21
    x, dy, coef, bias = _inputs(T, in_f, out_f, k, seed)
    xc, dyc, cc, bc = x.cuda(), dy.cuda(), coef.cuda(), bias.cuda()
    y = hip.linear_fwd(xc, cc, in_f, out_f, in_f, 1, seed, bias=bc)
    y_t = hip.linear_fwd(xc, cc, in_f, out_f, in_f, 1, seed, bias=bc, algo=RDB_ALGO_TILE)
    assert rel_l2(y.cpu().numpy(), y_t.cpu().numpy()) < F32_TOL
    dx = hip.linear_bwd_dx(dyc, cc, in_f, out_f, in_f, 1, seed)
    dx_t = hip.linear_bwd_dx(dyc, cc, in_f, out_f, in_f, 1, seed, algo=RDB_ALGO_TILE)
    assert rel_l2(dx.cpu().numpy(), dx_t.cpu().numpy()) < F32_TOL
    dc, _ = hip.linear_bwd_dcoef(dyc, xc, k, out_f, in_f, out_f, in_f, 1, seed)
    dc_t, _ = hip.linear_bwd_dcoef(dyc, xc, k, out_f, in_f, out_f, in_f, 1, seed, algo=RDB_ALGO_TILE)
    assert rel_l2(dc.cpu().numpy(), dc_t.cpu().numpy()) < F32_TOL


def test_strided_activations(hip, oracle):
    """x, dy, y's producers as column slices of wider matrices (leading dimension larger than the row)."""
    from randumb_amd._lib import RDB_ALGO_FACTORED

    T, in_f, out_f, k, seed = 260, 200, 328, 72, 13
    x, dy, coef, _ = _inputs(T, in_f, out_f, k, seed)
    wide_x = torch.zeros(T, in_f + 24).cuda()
    wide_x[:, 8:8 + in_f] = x.cuda()
    wide_dy = torch.zeros(T, out_f + 12).cuda()
    wide_dy[:, 4:4 + out_f] = dy.cuda()
    xs, dys, cc = wide_x[:, 8:8 + in_f], wide_dy[:, 4:4 + out_f], coef.cuda()
    assert not xs.is_contiguous() and not dys.is_contiguous()
    want_y = oracle.linear_fwd(x.numpy(), coef.numpy(), in_f, out_f, seed)
    want_dx, want_dc, _ = oracle.linear_bwd(x.numpy(), dy.numpy(), coef.numpy(), in_f, out_f, seed)
    y = hip.linear_fwd(xs, cc, in_f, out_f, in_f, 1, seed, algo=RDB_ALGO_FACTORED)
    assert rel_l2(y.cpu().numpy(), want_y) < F32_TOL
    dx = hip.linear_bwd_dx(dys, cc, in_f, out_f, in_f, 1, seed, algo=RDB_ALGO_FACTORED)
    assert rel_l2(dx.cpu().numpy(), want_dx) < F32_TOL
    dc, _ = hip.linear_bwd_dcoef(dys, xs, k, out_f, in_f, out_f, in_f, 1, seed, algo=RDB_ALGO_FACTORED)
    assert rel_l2(dc.cpu().numpy(), want_dc) < F32_TOL


def test_unaligned_views(hip, oracle):
    """Activations that start one element into a wider, odd-width matrix: neither the base nor the leading dimension is a
    multiple of 16 bytes."""
    from randumb_amd._lib import RDB_ALGO_FACTORED

    T, in_f, out_f, k, seed = 150, 96, 200, 72, 17
    x, dy, coef, bias = _inputs(T, in_f, out_f, k, seed)
    wide_x = torch.zeros(T, in_f + 3).cuda()
    wide_x[:, 1:1 + in_f] = x.cuda()
    wide_dy = torch.zeros(T, out_f + 5).cuda()
    wide_dy[:, 1:1 + out_f] = dy.cuda()
    xs, dys, cc = wide_x[:, 1:1 + in_f], wide_dy[:, 1:1 + out_f], coef.cuda()
    assert xs.data_ptr() % 16 and dys.data_ptr() % 16 and xs.stride(0) % 4 and dys.stride(0) % 4
    want_y = oracle.linear_fwd(x.numpy(), coef.numpy(), in_f, out_f, seed, bias=bias.numpy())
    want_dx, want_dc, _ = oracle.linear_bwd(x.numpy(), dy.numpy(), coef.numpy(), in_f, out_f, seed)
    y = hip.linear_fwd(xs, cc, in_f, out_f, in_f, 1, seed, bias=bias.cuda(), algo=RDB_ALGO_FACTORED)
    assert rel_l2(y.cpu().numpy(), want_y) < F32_TOL
    dx = hip.linear_bwd_dx(dys, cc, in_f, out_f, in_f, 1, seed, algo=RDB_ALGO_FACTORED)
    assert rel_l2(dx.cpu().numpy(), want_dx) < F32_TOL
    dc, _ = hip.linear_bwd_dcoef(dys, xs, k, out_f, in_f, out_f, in_f, 1, seed, algo=RDB_ALGO_FACTORED)
    assert rel_l2(dc.cpu().numpy(), want_dc) < F32_TOL


def test_layer_level_fp32(hip, oracle):
    """SillyLinear(matrix_coef=True) in fp32 at a GPT-like slice: forward, input gradient and coefficient gradient through autograd."""
    from randumb_amd.SillyLayers import SillyLinear

    T, in_f, out_f, k, seed = 1536, 256, 1024, 128, 4
    lin = SillyLinear(in_f, out_f, [k], [seed], bias=False, device="cuda", dtype=torch.float32, matrix_coef=True)
    g = torch.Generator().manual_seed(2)
    with torch.no_grad():
        lin.weight_coef.copy_((torch.randn(out_f, k, generator=g) * 0.01).cuda())
    x = torch.randn(T, in_f, generator=g)
    dy = torch.randn(T, out_f, generator=g)
    xc = x.cuda().requires_grad_(True)
    y = lin(xc)
    y.backward(dy.cuda())
    cn = lin.weight_coef.detach().cpu().numpy()
    want_y = oracle.linear_fwd(x.numpy(), cn, in_f, out_f, seed)
    want_dx, want_dc, _ = oracle.linear_bwd(x.numpy(), dy.numpy(), cn, in_f, out_f, seed)
    assert rel_l2(y.detach().cpu().numpy(), want_y) < F32_TOL
    assert rel_l2(xc.grad.cpu().numpy(), want_dx) < F32_TOL
    assert rel_l2(lin.weight_coef.grad.cpu().numpy(), want_dc) < F32_TOL


@pytest.mark.parametrize("T,in_f,out_f,k", [(1024, 768, 1024, 128), (200, 72, 136, 40), (1100, 1024, 260, 68), (333, 77, 55, 9)])
def test_fused_random_bias_in_fp32(hip, oracle, T, in_f, out_f, k):
    """W = C.N + s.noise1d (the reference's default layer, SillyLayers.py:122-133, 218-221) in fp32: forward, input gradient,
    coefficient gradient and the gradient of s against the oracle, with C != 0 and with C = 0; the gradient of s twice (same bits)."""
    print(f"case f32 random bias T={T} in={in_f} out={out_f} k={k}", flush=True)
    x, dy, coef, bias = _inputs(T, in_f, out_f, k, 31)
    sbv = 0.0625
    sb = torch.tensor([sbv])
    for c in (coef, torch.zeros_like(coef)):
        xn, dyn, cn = x.numpy(), dy.numpy(), c.numpy()
        want_y = oracle.linear_fwd(xn, cn, in_f, out_f, 9, bias=bias.numpy(), scale_bias=sbv)
        want_dx, want_dc, dW = oracle.linear_bwd(xn, dyn, cn, in_f, out_f, 9, scale_bias=sbv)
        want_ds = float(oracle.scale_bias_bwd(dW.astype(np.float32), 9)[0])
        xg, dyg, cg, sg = x.cuda(), dy.cuda(), c.cuda(), sb.cuda()
        y = hip.linear_fwd(xg, cg, in_f, out_f, in_f, 1, 9, scale_bias=sg, bias=bias.cuda())
        dx = hip.linear_bwd_dx(dyg, cg, in_f, out_f, in_f, 1, 9, scale_bias=sg)
        dc, ds = hip.linear_bwd_dcoef(dyg, xg, k, out_f, in_f, out_f, in_f, 1, 9, want_scale_bias_grad=True)
        assert rel_l2(y.cpu().numpy(), want_y) < F32_TOL
        assert rel_l2(dx.cpu().numpy(), want_dx) < F32_TOL
        assert rel_l2(dc.cpu().numpy(), want_dc) < F32_TOL
        assert abs(float(ds) - want_ds) < 1e-4 * max(abs(want_ds), float(np.linalg.norm(dW)))
        _, ds2 = hip.linear_bwd_dcoef(dyg, xg, k, out_f, in_f, out_f, in_f, 1, 9, want_scale_bias_grad=True)
        assert torch.equal(ds, ds2)


@pytest.mark.parametrize("rows,row_len,k", [(512, 768, 256), (300, 1001, 230), (2048, 260, 132)])
def test_materialise_on_the_matrix_cores(hip, oracle, rows, row_len, k):
    """Matrix-coef W = C.N (+ s.noise1d) written to memory, its transposed view, and the adjoint dcoef = dW.N^T, at sizes the
    matrix-core kernels take (some tens of millions of multiply-adds on), against the oracle."""
    print(f"case materialise on the matrix cores rows={rows} row_len={row_len} k={k}", flush=True)
    g = torch.Generator().manual_seed(rows + k)
    C = torch.randn(rows, k, generator=g) * 0.05
    sb = torch.tensor([0.3])
    for s_ in (None, sb):
        sbv = None if s_ is None else 0.3
        W = oracle.materialize_fwd(C.numpy(), (rows, row_len), (row_len, 1), 7, scale_bias=sbv, row_len=row_len)
        got = hip.materialize_fwd(C.cuda(), (rows, row_len), (row_len, 1), 7, None if s_ is None else s_.cuda(), s_ is not None, row_len)
        assert got.shape == (rows, row_len) and rel_l2(got.cpu().numpy(), W) < F32_TOL
        got_t = hip.materialize_fwd(C.cuda(), (row_len, rows), (1, row_len), 7, None if s_ is None else s_.cuda(), s_ is not None, row_len)
        assert got_t.shape == (row_len, rows) and rel_l2(got_t.cpu().numpy(), W.T) < F32_TOL
    dW = torch.randn(rows, row_len, generator=g)
    want = oracle.materialize_bwd(dW.numpy(), k, 7, coef_rows=rows)
    got = hip.materialize_bwd(dW.cuda(), k, 7, rows)
    assert got.shape == (rows, k) and rel_l2(got.cpu().numpy(), want) < F32_TOL
    got2 = hip.materialize_bwd(dW.cuda(), k, 7, rows)
    assert torch.equal(got, got2)


@pytest.mark.parametrize("T,in_f,out_f,k,seed", [s for s in SHAPES if s[0] != 4500] + [(2500, 200, 96, 160, 4)])
def test_projected_form_in_fp32(hip, oracle, T, in_f, out_f, k, seed):
    """The state-saving form of an fp32 layer: the forward call leaves z = x . N^T (fp32) in the state, the backward call takes
    dx and dC from dy, the state and C without x.  Against the oracle at 1e-5; z itself against x @ Noise.T; the coefficient
    gradient alone (dx not wanted) gives the bits of the full call; the same call twice gives the same bits.  The last shape
    has k > out_f: the projection's contraction ranges find no room in y and run as one range."""
    print(f"case f32 projected T={T} in={in_f} out={out_f} k={k}", flush=True)
    x, dy, coef, bias = _inputs(T, in_f, out_f, k, seed)
    xn, dyn, cn = x.numpy(), dy.numpy(), coef.numpy()
    want_y = oracle.linear_fwd(xn, cn, in_f, out_f, seed, bias=bias.numpy())
    want_dx, want_dc, _ = oracle.linear_bwd(xn, dyn, cn, in_f, out_f, seed)
    xc, dyc, cc = x.cuda(), dy.cuda(), coef.cuda()
    assert hip.linear_projection_supported(T, in_f, out_f, k, torch.float32)
    y, state = hip.linear_project_fwd(xc, cc, seed, bias=bias.cuda())
    assert y.dtype == torch.float32 and rel_l2(y.cpu().numpy(), want_y) < F32_TOL
    z = hip.projection_unpack(state, in_f, out_f, k, torch.float32)["z"]
    noise = oracle.noise_2d(in_f, k, seed).astype(np.float64)   # [i, m]
    assert rel_l2(z.cpu().numpy(), xn.astype(np.float64) @ noise) < F32_TOL
    dx, dc = hip.linear_bwd_projected(dyc, state, cc, in_f, seed)
    assert dx.dtype == torch.float32 and rel_l2(dx.cpu().numpy(), want_dx) < F32_TOL
    assert dc.dtype == torch.float32 and rel_l2(dc.cpu().numpy(), want_dc) < F32_TOL
    none, dc_only = hip.linear_bwd_projected(dyc, state, cc, in_f, seed, want_dx=False)
    assert none is None and torch.equal(dc_only, dc)
    dx2, dc2 = hip.linear_bwd_projected(dyc, state, cc, in_f, seed)
    assert torch.equal(dx2, dx) and torch.equal(dc2, dc)
    # the state serves the separate forward call too, and the projection alone (one contraction range) agrees to rounding
    y2 = hip.linear_fwd_projected(state, cc, in_f, seed, bias=bias.cuda(), f32_state=True)
    assert torch.equal(y2, y)
    state1 = hip.linear_project(xc, k, out_f, seed)
    z1 = hip.projection_unpack(state1, in_f, out_f, k, torch.float32)["z"]
    assert rel_l2(z1.cpu().numpy(), z.cpu().numpy()) < 1e-6


def test_fp32_layer_takes_the_projected_form(hip, oracle):
    """SillyLinear in fp32 beyond the few-token regime saves z for the backward pass (ops.linear's choice) and matches the oracle."""
    import randumb_amd as ra
    from randumb_amd import ops

    T, in_f, out_f, k, seed = 1500, 264, 520, 136, 31
    assert hip.linear_projection_preferred(T, in_f, out_f, k, torch.float32)
    assert not hip.linear_projection_preferred(128, 784, 256, 64, torch.float32)   # the few-token regime keeps its own kernels
    layer = ra.SillyLinear(in_f, out_f, [k, k], [seed, seed + 1], bias=False, matrix_coef=True).cuda()
    x, dy, coef, _ = _inputs(T, in_f, out_f, k, seed)
    with torch.no_grad():
        layer.weight_coef.copy_(coef)
        layer.weight_scale_bias.zero_()
    seen = []
    orig = ops._ProjectedLinear.apply
    try:
        ops._ProjectedLinear.apply = staticmethod(lambda *a: (seen.append(1), orig(*a))[1])
        xg = x.cuda().requires_grad_()
        y = layer(xg)
        y.backward(dy.cuda())
    finally:
        ops._ProjectedLinear.apply = orig
    assert seen, "the fp32 layer did not take the projected form"
    want_y = oracle.linear_fwd(x.numpy(), coef.numpy(), in_f, out_f, seed)
    want_dx, want_dc, _ = oracle.linear_bwd(x.numpy(), dy.numpy(), coef.numpy(), in_f, out_f, seed)
    assert rel_l2(y.detach().cpu().numpy(), want_y) < F32_TOL
    assert rel_l2(xg.grad.cpu().numpy(), want_dx) < F32_TOL
    assert rel_l2(layer.weight_coef.grad.cpu().numpy(), want_dc) < F32_TOL
    # the first layer of a network: its input needs no gradient
    layer.zero_grad()
    layer(x.cuda()).backward(dy.cuda())
    assert rel_l2(layer.weight_coef.grad.cpu().numpy(), want_dc) < F32_TOL


@pytest.mark.parametrize("T,in_f,out_f,k,seed", [(512, 768, 1024, 128, 3), (333, 777, 555, 99, 8), (2100, 516, 132, 100, 77)])
def test_split_products_are_as_accurate_as_fp32_instructions(hip, oracle, T, in_f, out_f, k, seed):
    """rdb_set_f32_split: the same calls with the operands split three ways onto the bf16 matrix instructions (default) and on
    the fp32 matrix instructions.  Both within the fp32 tolerance of the fp64 oracle, the split products no further from it than
    1.5 times the fp32 instructions' own error (plus a floor), and the two a few fp32 roundings apart.  Inputs with a wide
    range of magnitudes, so that the low parts matter."""
    from randumb_amd._lib import RDB_ALGO_FACTORED

    print(f"case f32 split vs fp32 instructions T={T} in={in_f} out={out_f} k={k}", flush=True)
    x, dy, coef, bias = _inputs(T, in_f, out_f, k, seed)
    g = torch.Generator().manual_seed(seed + 100)
    x = x * torch.exp(3.0 * torch.randn(T, 1, generator=g))          # rows of very different sizes
    coef = coef * torch.exp(2.0 * torch.randn(1, k, generator=g))
    xn, dyn, cn = x.numpy(), dy.numpy(), coef.numpy()
    want_y = oracle.linear_fwd(xn, cn, in_f, out_f, seed, bias=bias.numpy())
    want_dx, want_dc, _ = oracle.linear_bwd(xn, dyn, cn, in_f, out_f, seed)
    xg, dyg, cg, bg = x.cuda(), dy.cuda(), coef.cuda(), bias.cuda()
    got = {}
    before = hip.set_f32_split(1)
    try:
        for mode in (1, 0):
            hip.set_f32_split(mode)
            y = hip.linear_fwd(xg, cg, in_f, out_f, in_f, 1, seed, bias=bg, algo=RDB_ALGO_FACTORED)
            dx = hip.linear_bwd_dx(dyg, cg, in_f, out_f, in_f, 1, seed, algo=RDB_ALGO_FACTORED)
            dc, _ = hip.linear_bwd_dcoef(dyg, xg, k, out_f, in_f, out_f, in_f, 1, seed, algo=RDB_ALGO_FACTORED)
            got[mode] = [t.cpu().numpy() for t in (y, dx, dc)]
    finally:
        hip.set_f32_split(before)
    for name, i, want in (("y", 0, want_y), ("dx", 1, want_dx), ("dcoef", 2, want_dc)):
        e_split, e_f32 = rel_l2(got[1][i], want), rel_l2(got[0][i], want)
        print(f"  {name}: split {e_split:.2e}  fp32 instructions {e_f32:.2e}  between them {rel_l2(got[1][i], got[0][i]):.2e}", flush=True)
        assert e_split < F32_TOL and e_f32 < F32_TOL, name
        assert e_split < 1.5 * e_f32 + 2e-7, name
        assert rel_l2(got[1][i], got[0][i]) < 2e-6, name
