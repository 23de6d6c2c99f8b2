"""GPU parity of the HIP kernels (called through the C ABI) against the CPU oracle.

Integer/noise results must be bit-exact.  Floating-point tolerances (relative L2 norm):
fp32 paths 1e-5, bf16 paths 2e-2 - the bounds the task states for this path.
"""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

F32_TOL = 1e-5
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


def cpu(t):
    return t.detach().float().cpu().numpy()


# ------------------------------------------------------------------------------------------------ noise
@pytest.mark.parametrize("N,M,seed", [(1, 1, 0), (3, 6, 1337), (1000, 257, 47), (4096, 16, 2**31 - 1), (70, 1024, 0xFFFFFFFF)])
def test_noise_2d_bit_exact(hip, oracle, N, M, seed):
    print(f"case noise2d N={N} M={M} seed={seed}", flush=True)
    got = cpu(hip.sq5_fill_2d(N, M, seed))
    want = oracle.noise_2d(N, M, seed)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))


def test_noise_2d_wraparound_rows_bit_exact(hip, oracle):
    # rows whose PRIME*n product wraps 2**32 many times: compare the tail of a tall matrix
    N, M, seed = 3_000_000, 4, 1337
    print("case noise2d tall", flush=True)
    got = cpu(hip.sq5_fill_2d(N, M, seed)[-1000:])
    want = oracle.noise_2d_np(np.arange(N - 1000, N), np.arange(M), seed)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))


@pytest.mark.parametrize("N,seed", [(1, 0), (1000003, 1337)])
def test_noise_1d_bit_exact(hip, oracle, N, seed):
    got = cpu(hip.sq5_fill_1d(N, seed))
    assert np.array_equal(got.view(np.uint32), oracle.noise_1d(N, seed).view(np.uint32))


def test_empty_shapes(hip):
    assert hip.sq5_fill_2d(0, 5, 1).shape == (0, 5)
    assert hip.sq5_fill_1d(0, 1).shape == (0,)
    c = torch.randn(4, device="cuda")
    assert hip.materialize_fwd(c, (0, 3), (3, 1), 1, None, False).shape == (0, 3)


# ------------------------------------------------------------------------------------------------ materialise
@pytest.mark.parametrize("P,Q,k,seed", [(3, 6, 18, 1337), (256, 784, 64, 1337), (10, 256, 64, 1338), (1, 37, 5, 0), (129, 65, 2049, 3)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_materialize_fwd_vector_coef(hip, oracle, P, Q, k, seed, dtype):
    print(f"case mat_fwd vec P={P} Q={Q} k={k} {dtype}", flush=True)
    g = torch.Generator().manual_seed(0)
    c = torch.randn(k, generator=g).to(dtype)
    sb = torch.tensor([0.37]).to(dtype)
    for fused in (False, True):
        got = cpu(hip.materialize_fwd(c.cuda(), (P, Q), (Q, 1), seed, sb.cuda() if fused else None, fused))
        want = oracle.materialize_fwd(c.float().numpy(), (P, Q), (Q, 1), seed, float(sb.float()) if fused else None)
        assert got.dtype == np.float32 and rel_l2(got, want) < F32_TOL
    # transposed view: same values, transposed
    got_t = cpu(hip.materialize_fwd(c.cuda(), (Q, P), (1, Q), seed, None, False))
    got = cpu(hip.materialize_fwd(c.cuda(), (P, Q), (Q, 1), seed, None, False))
    assert np.array_equal(got_t, got.T)


def test_materialize_fwd_unit_coef_is_noise_bit_exact(hip, oracle):
    P, Q, k, seed = 33, 65, 40, 1337
    noise = oracle.noise_2d(P * Q, k, seed)
    for j in (0, 17, 39):
        c = torch.zeros(k)
        c[j] = 1.0
        got = cpu(hip.materialize_fwd(c.cuda(), (P, Q), (Q, 1), seed, None, False)).reshape(-1)
        assert np.array_equal(got, noise[:, j])
    one_d = cpu(hip.materialize_fwd(c.cuda(), (Q,), (1,), seed, None, False))
    assert np.array_equal(one_d, noise[:Q, 39])


@pytest.mark.parametrize("out_f,in_f,k,seed", [(7, 13, 24, 47), (256, 784, 64, 1337), (10, 256, 64, 1338), (100, 200, 33, 5)])
def test_materialize_fwd_matrix_coef(hip, oracle, out_f, in_f, k, seed):
    print(f"case mat_fwd mat out={out_f} in={in_f} k={k}", flush=True)
    g = torch.Generator().manual_seed(1)
    C = torch.randn(out_f, k, generator=g)
    sb = torch.tensor([0.5])
    want = oracle.materialize_fwd(C.numpy(), (out_f, in_f), (in_f, 1), seed, row_len=in_f)
    got = cpu(hip.materialize_fwd(C.cuda(), (out_f, in_f), (in_f, 1), seed, None, False))
    assert rel_l2(got, want) < F32_TOL
    got_t = cpu(hip.materialize_fwd(C.cuda(), (in_f, out_f), (1, in_f), seed, None, False))
    assert np.array_equal(got_t, got.T)
    want_b = oracle.materialize_fwd(C.numpy(), (out_f, in_f), (in_f, 1), seed, 0.5, row_len=in_f)
    got_b = cpu(hip.materialize_fwd(C.cuda(), (out_f, in_f), (in_f, 1), seed, sb.cuda(), True))
    assert rel_l2(got_b, want_b) < F32_TOL
    # a view that is neither the base nor its transpose goes through the per-element kernel: first two rows only
    got_v = cpu(hip.materialize_fwd(C.cuda(), (2, in_f), (in_f, 1), seed, None, False, row_len=in_f))
    assert rel_l2(got_v, want[:2]) < F32_TOL


@pytest.mark.parametrize("Nw,k,seed", [(18, 18, 1337), (200704, 64, 1337), (2560, 64, 1338), (5000, 300, 9), (1, 7, 0)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_materialize_bwd_vector_coef(hip, oracle, Nw, k, seed, dtype):
    print(f"case mat_bwd vec Nw={Nw} k={k} {dtype}", flush=True)
    g = torch.Generator().manual_seed(2)
    d = torch.randn(Nw, generator=g).to(dtype)
    got = cpu(hip.materialize_bwd(d.cuda(), k, seed))
    want = oracle.materialize_bwd(d.float().numpy(), k, seed)
    assert got.shape == (k,) and rel_l2(got, want) < F32_TOL
    again = cpu(hip.materialize_bwd(d.cuda(), k, seed))
    assert np.array_equal(got, again)  # fixed reduction tree: reproducible


def test_materialize_bwd_unit_vector_bit_exact(hip, oracle):
    Nw, k, seed = 5000, 70, 1337
    noise = oracle.noise_2d(Nw, k, seed)
    for n in (0, 2049, Nw - 1):
        d = torch.zeros(Nw)
        d[n] = 1.0
        assert np.array_equal(cpu(hip.materialize_bwd(d.cuda(), k, seed)), noise[n])


@pytest.mark.parametrize("out_f,in_f,k,seed", [(7, 13, 24, 47), (256, 784, 64, 1337), (100, 200, 33, 5)])
def test_materialize_bwd_matrix_coef(hip, oracle, out_f, in_f, k, seed):
    g = torch.Generator().manual_seed(3)
    d = torch.randn(out_f, in_f, generator=g)
    got = cpu(hip.materialize_bwd(d.cuda(), k, seed, coef_rows=out_f))
    want = oracle.materialize_bwd(d.numpy(), k, seed, coef_rows=out_f)
    assert got.shape == (out_f, k) and rel_l2(got, want) < F32_TOL


@pytest.mark.parametrize("Nw", [1, 501, 300000])
def test_scale_bias_bwd(hip, oracle, Nw):
    g = torch.Generator().manual_seed(4)
    d = torch.randn(Nw, generator=g)
    got = cpu(hip.scale_bias_bwd(d.cuda(), 77))
    want = oracle.scale_bias_bwd(d.numpy(), 77)
    assert got.shape == (1,) and abs(got[0] - want[0]) < 1e-4 * max(1.0, abs(want[0]))


def test_embedding(hip, oracle):
    g = torch.Generator().manual_seed(5)
    rows, rowsize, k, seed = 50304, 768, 32, 1337
    c = torch.randn(k, generator=g)
    idx = torch.randint(0, rows, (3, 17), generator=g)
    idx[0, 0], idx[0, 1] = rows - 1, rows - 1  # repeated index, last row
    got = cpu(hip.embed_fwd(idx.cuda(), c.cuda(), rowsize, seed))
    want = oracle.embed_fwd(idx.numpy(), c.numpy(), rowsize, seed)
    assert got.shape == (3, 17, rowsize) and rel_l2(got, want) < F32_TOL
    D = torch.randn(3, 17, rowsize, generator=g)
    gotb = cpu(hip.embed_bwd(idx.cuda(), D.cuda(), k, rowsize, seed))
    wantb = oracle.embed_bwd(idx.numpy(), D.numpy(), k, rowsize, seed)
    assert rel_l2(gotb, wantb) < F32_TOL


# ------------------------------------------------------------------------------------------------ fused linear
LIN_SHAPES = [
    # tokens, in_f, out_f, k, seed
    (9, 12, 5, 18, 1337),
    (128, 784, 256, 64, 1337),   # MNIST-shaped layer 1
    (128, 256, 10, 64, 1338),    # MNIST-shaped layer 2
    (200, 100, 130, 40, 7),      # ragged everything
    (256, 768, 384, 256, 0),     # a slice of the GPT-2 MLP shape
]


def _inputs(T, in_f, out_f, k, matrix, dtype, seed):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(T, in_f, generator=g).to(dtype)
    dy = torch.randn(T, out_f, generator=g).to(dtype)
    std = (3.0 / k) ** 0.5 * 0.05
    coef = (torch.randn((out_f, k) if matrix else (k,), generator=g) * std).to(dtype)
    return x, dy, coef


@pytest.mark.parametrize("T,in_f,out_f,k,seed", LIN_SHAPES)
@pytest.mark.parametrize("matrix", [True, False])
@pytest.mark.parametrize("dtype,tol", [(torch.float32, F32_TOL), (torch.bfloat16, BF16_TOL)])
def test_linear_fwd_bwd(hip, oracle, T, in_f, out_f, k, seed, matrix, dtype, tol):
    print(f"case linear T={T} in={in_f} out={out_f} k={k} matrix={matrix} {dtype}", flush=True)
    x, dy, coef = _inputs(T, in_f, out_f, k, matrix, dtype, seed)
    xn, dyn, cn = x.float().numpy(), dy.float().numpy(), coef.float().numpy()
    want_y = oracle.linear_fwd(xn, cn, in_f, out_f, seed)
    want_dx, want_dc, _ = oracle.linear_bwd(xn, dyn, cn, in_f, out_f, seed)
    xc, dyc, cc = x.cuda(), dy.cuda(), coef.cuda()
    y = hip.linear_fwd(xc, cc, in_f, out_f, in_f, 1, seed)
    assert y.dtype == dtype and y.shape == (T, out_f)
    assert rel_l2(cpu(y), want_y) < tol
    dx = hip.linear_bwd_dx(dyc, cc, in_f, out_f, in_f, 1, seed)
    assert dx.dtype == dtype and rel_l2(cpu(dx), want_dx) < tol
    dc, dsb = hip.linear_bwd_dcoef(dyc, xc, k, out_f if matrix else 0, in_f, out_f, in_f, 1, seed)
    assert dsb is None and dc.dtype == torch.float32 and dc.shape == coef.shape
    assert rel_l2(cpu(dc), want_dc) < tol


def test_linear_bias_and_scale_bias(hip, oracle):
    T, in_f, out_f, k, seed = 64, 96, 48, 32, 1337
    for matrix in (True, False):
        x, dy, coef = _inputs(T, in_f, out_f, k, matrix, torch.float32, 11)
        bias = torch.randn(out_f)
        sb = torch.tensor([0.02])
        want = oracle.linear_fwd(x.numpy(), coef.numpy(), in_f, out_f, seed, bias=bias.numpy(), scale_bias=0.02)
        got = hip.linear_fwd(x.cuda(), coef.cuda(), in_f, out_f, in_f, 1, seed, scale_bias=sb.cuda(), bias=bias.cuda())
        assert rel_l2(cpu(got), want) < F32_TOL
        want_dx, want_dc, dW = oracle.linear_bwd(x.numpy(), dy.numpy(), coef.numpy(), in_f, out_f, seed, scale_bias=0.02)
        dx = hip.linear_bwd_dx(dy.cuda(), coef.cuda(), in_f, out_f, in_f, 1, seed, scale_bias=sb.cuda())
        assert rel_l2(cpu(dx), want_dx) < F32_TOL
        dc, dsb = hip.linear_bwd_dcoef(dy.cuda(), x.cuda(), k, out_f if matrix else 0, in_f, out_f, in_f, 1, seed,
                                       want_scale_bias_grad=True)
        assert rel_l2(cpu(dc), want_dc) < F32_TOL
        want_ds = oracle.scale_bias_bwd(dW.astype(np.float32), seed)
        assert abs(cpu(dsb)[0] - want_ds[0]) < 1e-4 * max(1.0, abs(want_ds[0]))


def test_linear_strided_weight_vector_coef(hip, oracle):
    """`mat1 @ tensor` with a contiguous (P, Q) tensor: out_f = Q, in_f = P, strides (1, Q)  (rt_mm's case)."""
    L, P, Q, k, seed = 40, 24, 36, 16, 1337
    g = torch.Generator().manual_seed(6)
    mat1 = torch.randn(L, P, generator=g)
    c = torch.randn(k, generator=g)
    W = oracle.materialize_fwd(c.numpy(), (P, Q), (Q, 1), seed).astype(np.float64)
    got = hip.linear_fwd(mat1.cuda(), c.cuda(), P, Q, 1, Q, seed)
    assert rel_l2(cpu(got), mat1.double().numpy() @ W) < F32_TOL


@pytest.mark.parametrize("dtype,tol", [(torch.float32, 2e-6), (torch.bfloat16, 1e-2)])
def test_vector_coef_split_form_against_the_general_kernel(hip, dtype, tol):
    """The vector-coef forward and input gradient whose blocks own tiles of W (AUTO, with the workspace the library asks for)
    against the general kernel that owns tiles of the output (RDB_ALGO_TILE): the same W bits, sums in another order.  Ragged
    sizes, more than one token tile, fused random bias, bias; the same call twice gives the same bits."""
    from randumb_amd._lib import RDB_ALGO_TILE

    T, in_f, out_f, k, seed = 300, 200, 136, 72, 11
    g = torch.Generator().manual_seed(3)
    x = torch.randn(T, in_f, generator=g).to(dtype).cuda()
    dy = torch.randn(T, out_f, generator=g).to(dtype).cuda()
    c = (torch.randn(k, generator=g) * 0.05).to(dtype).cuda()
    sb = torch.tensor([0.07]).to(dtype).cuda()
    bias = torch.randn(out_f, generator=g).to(dtype).cuda()
    rel = lambda a, b: float((a.float() - b.float()).norm() / b.float().norm())
    for scale_bias in (None, sb):
        y = hip.linear_fwd(x, c, in_f, out_f, in_f, 1, seed, scale_bias=scale_bias, bias=bias)
        y_t = hip.linear_fwd(x, c, in_f, out_f, in_f, 1, seed, scale_bias=scale_bias, bias=bias, algo=RDB_ALGO_TILE)
        assert rel(y, y_t) < tol
        assert torch.equal(y, hip.linear_fwd(x, c, in_f, out_f, in_f, 1, seed, scale_bias=scale_bias, bias=bias))
        dx = hip.linear_bwd_dx(dy, c, in_f, out_f, in_f, 1, seed, scale_bias=scale_bias)
        dx_t = hip.linear_bwd_dx(dy, c, in_f, out_f, in_f, 1, seed, scale_bias=scale_bias, algo=RDB_ALGO_TILE)
        assert rel(dx, dx_t) < tol
        assert torch.equal(dx, hip.linear_bwd_dx(dy, c, in_f, out_f, in_f, 1, seed, scale_bias=scale_bias))
        # the coefficient gradient with room for dW in the workspace (dW formed once, contracted once with its k hashed values per
        # element) against the general kernel, with and without the gradient of the random bias's scale
        want_ds = scale_bias is not None
        dc, ds = hip.linear_bwd_dcoef(dy, x, k, 0, in_f, out_f, in_f, 1, seed, want_scale_bias_grad=want_ds)
        dc_t, ds_t = hip.linear_bwd_dcoef(dy, x, k, 0, in_f, out_f, in_f, 1, seed, want_scale_bias_grad=want_ds, algo=RDB_ALGO_TILE)
        assert rel(dc, dc_t) < max(tol, 1e-5)
        again = hip.linear_bwd_dcoef(dy, x, k, 0, in_f, out_f, in_f, 1, seed, want_scale_bias_grad=want_ds)
        assert torch.equal(dc, again[0])
        if want_ds:
            assert abs(float(ds) - float(ds_t)) < max(tol, 1e-5) * max(1.0, abs(float(ds_t))) and torch.equal(ds, again[1])


def test_argument_errors(hip):
    from randumb_amd._lib import RandumbHipError

    x = torch.randn(4, 8, device="cuda")
    C = torch.randn(6, 3, device="cuda")
    with pytest.raises(RandumbHipError):  # matrix-coef with a transposed weight layout
        hip.linear_fwd(x, C, 8, 6, 1, 6, 0)
    with pytest.raises(ValueError):
        hip.sq5_fill_1d(4, -1)
    with pytest.raises(NotImplementedError):
        hip.materialize_fwd(torch.randn(4), (2, 2), (2, 1), 0, None, False)


# ------------------------------------------------------------------------------------------------ strip-stationary forward
STRIP_SHAPES = [
    # tokens, in_f, out_f, k, seed
    (1024, 768, 3072, 256, 0),   # full-width slice of the GPT-2 MLP shape (96-row strips)
    (1000, 768, 200, 256, 3),    # ragged tokens and a ragged last strip
    (77, 72, 130, 40, 7),        # in_f not a multiple of 64, k not a multiple of 16
    (4096, 1536, 96, 64, 11),    # 32-row strips (a 64-row strip of 1536 columns does not fit next to nothing else)
    (33, 8, 5, 3, 1),
]


@pytest.mark.parametrize("T,in_f,out_f,k,seed", STRIP_SHAPES)
@pytest.mark.parametrize("coef_dtype", [torch.bfloat16, torch.float32])
def test_linear_fwd_strip_algorithm(hip, oracle, T, in_f, out_f, k, seed, coef_dtype):
    from randumb_amd._lib import RDB_ALGO_STRIP, RDB_ALGO_TILE

    print(f"case strip T={T} in={in_f} out={out_f} k={k} coef={coef_dtype}", flush=True)
    x, _, coef = _inputs(T, in_f, out_f, k, True, torch.bfloat16, seed)
    coef = coef.float().to(coef_dtype)
    bias = torch.randn(out_f).bfloat16()
    sb = torch.tensor([0.01]).to(coef_dtype)
    want = oracle.linear_fwd(x.float().numpy(), coef.float().numpy(), in_f, out_f, seed)
    got = hip.linear_fwd(x.cuda(), coef.cuda(), in_f, out_f, in_f, 1, seed, algo=RDB_ALGO_STRIP)
    assert got.shape == (T, out_f) and rel_l2(cpu(got), want) < BF16_TOL
    ref = hip.linear_fwd(x.cuda(), coef.cuda(), in_f, out_f, in_f, 1, seed, algo=RDB_ALGO_TILE)
    assert rel_l2(cpu(got), cpu(ref)) < 5e-3  # two on-chip schedules of the same bf16 arithmetic
    want_b = oracle.linear_fwd(x.float().numpy(), coef.float().numpy(), in_f, out_f, seed, bias=bias.float().numpy(),
                               scale_bias=float(sb.float()))
    got_b = hip.linear_fwd(x.cuda(), coef.cuda(), in_f, out_f, in_f, 1, seed, scale_bias=sb.cuda(), bias=bias.cuda(),
                           algo=RDB_ALGO_STRIP)
    assert rel_l2(cpu(got_b), want_b) < BF16_TOL


def test_strip_algorithm_rejects_what_it_cannot_do(hip):
    from randumb_amd._lib import RandumbHipError, RDB_ALGO_STRIP

    x = torch.randn(64, 100, device="cuda").bfloat16()   # in_f not a multiple of 8
    C = torch.randn(32, 16, device="cuda").bfloat16()
    with pytest.raises(RandumbHipError):
        hip.linear_fwd(x, C, 100, 32, 100, 1, 0, algo=RDB_ALGO_STRIP)
    assert hip.linear_fwd(x, C, 100, 32, 100, 1, 0).shape == (64, 32)  # the default falls back to the general kernel


# ------------------------------------------------------------------------------------------------ optimised backward kernels
BWD_SHAPES = [
    # tokens, in_f, out_f, k, seed
    (2048, 768, 3072, 256, 0),   # a quarter of the headline workload
    (1000, 200, 328, 72, 3),     # ragged against every tile size (multiples of 8 only)
    (64, 8, 8, 8, 5),
    (520, 136, 200, 248, 11),    # k = 8 mod 16, a partial chunk of output rows, three token tiles
    (300, 1024, 96, 512, 9),     # k larger than in*out/(in+out): the factored form is not cheaper, still exact when forced
]


@pytest.mark.parametrize("T,in_f,out_f,k,seed", BWD_SHAPES)
def test_linear_bwd_fast_kernels(hip, oracle, T, in_f, out_f, k, seed):
    from randumb_amd._lib import RandumbHipError, RDB_ALGO_FACTORED, RDB_ALGO_STRIP, RDB_ALGO_TILE

    print(f"case bwd fast T={T} in={in_f} out={out_f} k={k}", flush=True)
    x, dy, coef = _inputs(T, in_f, out_f, k, True, torch.bfloat16, seed)
    want_dx, want_dc, dW = oracle.linear_bwd(x.float().numpy(), dy.float().numpy(), coef.float().numpy(), in_f, out_f, seed)
    xc, dyc, cc = x.cuda(), dy.cuda(), coef.cuda()
    dx = hip.linear_bwd_dx(dyc, cc, in_f, out_f, in_f, 1, seed, algo=RDB_ALGO_FACTORED)
    assert dx.shape == (T, in_f) and rel_l2(cpu(dx), want_dx) < BF16_TOL
    dx_ref = hip.linear_bwd_dx(dyc, cc, in_f, out_f, in_f, 1, seed, algo=RDB_ALGO_TILE)
    assert rel_l2(cpu(dx), cpu(dx_ref)) < 1e-2
    assert rel_l2(cpu(hip.linear_bwd_dx(dyc, cc, in_f, out_f, in_f, 1, seed)), want_dx) < BF16_TOL  # whatever AUTO picks
    if k <= 256:   # the kernel that forms W chunks on chip from a noise strip kept in LDS
        dx_s = hip.linear_bwd_dx(dyc, cc, in_f, out_f, in_f, 1, seed, algo=RDB_ALGO_STRIP)
        assert dx_s.shape == (T, in_f) and rel_l2(cpu(dx_s), want_dx) < BF16_TOL
        assert rel_l2(cpu(dx_s), cpu(dx_ref)) < 1e-2
    else:
        with pytest.raises(RandumbHipError, match="strip algorithm"):
            hip.linear_bwd_dx(dyc, cc, in_f, out_f, in_f, 1, seed, algo=RDB_ALGO_STRIP)
    dc, dsb = hip.linear_bwd_dcoef(dyc, xc, k, out_f, in_f, out_f, in_f, 1, seed, want_scale_bias_grad=True)
    assert rel_l2(cpu(dc), want_dc) < BF16_TOL
    dc_ref, _ = hip.linear_bwd_dcoef(dyc, xc, k, out_f, in_f, out_f, in_f, 1, seed, algo=RDB_ALGO_TILE)
    assert rel_l2(cpu(dc), cpu(dc_ref)) < 1e-2
    dc_f, _ = hip.linear_bwd_dcoef(dyc, xc, k, out_f, in_f, out_f, in_f, 1, seed, algo=RDB_ALGO_FACTORED)
    assert dc_f.shape == (out_f, k) and rel_l2(cpu(dc_f), want_dc) < BF16_TOL
    dc_s, _ = hip.linear_bwd_dcoef(dyc, xc, k, out_f, in_f, out_f, in_f, 1, seed, algo=RDB_ALGO_STRIP)   # dW-tile kernel
    assert rel_l2(cpu(dc_s), want_dc) < BF16_TOL
    dc_a, _ = hip.linear_bwd_dcoef(dyc, xc, k, out_f, in_f, out_f, in_f, 1, seed)
    assert rel_l2(cpu(dc_a), want_dc) < BF16_TOL
    # forward: factored vs the oracle, vs the weight-forming kernel, with and without bias
    want_y = oracle.linear_fwd(x.float().numpy(), coef.float().numpy(), in_f, out_f, seed)
    y_f = hip.linear_fwd(xc, cc, in_f, out_f, in_f, 1, seed, algo=RDB_ALGO_FACTORED)
    assert y_f.shape == (T, out_f) and rel_l2(cpu(y_f), want_y) < BF16_TOL
    y_t = hip.linear_fwd(xc, cc, in_f, out_f, in_f, 1, seed, algo=RDB_ALGO_TILE)
    assert rel_l2(cpu(y_f), cpu(y_t)) < 1e-2
    bias = torch.randn(out_f).bfloat16()
    want_yb = oracle.linear_fwd(x.float().numpy(), coef.float().numpy(), in_f, out_f, seed, bias=bias.float().numpy())
    assert rel_l2(cpu(hip.linear_fwd(xc, cc, in_f, out_f, in_f, 1, seed, bias=bias.cuda(), algo=RDB_ALGO_FACTORED)), want_yb) < BF16_TOL
    assert rel_l2(cpu(hip.linear_fwd(xc, cc, in_f, out_f, in_f, 1, seed, bias=bias.cuda())), want_yb) < BF16_TOL
    want_ds = float(oracle.scale_bias_bwd(dW.astype(np.float32), seed)[0])
    assert abs(float(dsb) - want_ds) < 2e-2 * max(1.0, abs(want_ds), float(np.abs(dW).sum()) ** 0.5)


@pytest.mark.parametrize("T,in_f,out_f,k,seed", BWD_SHAPES)
def test_linear_projected_form(hip, oracle, T, in_f, out_f, k, seed):
    """z = x.N^T once, then y = z.C^T and dcoef = dy^T.z from it: same results as the one-call entry points."""
    print(f"case projected T={T} in={in_f} out={out_f} k={k}", flush=True)
    x, dy, coef = _inputs(T, in_f, out_f, k, True, torch.bfloat16, seed)
    xn, dyn, cn = x.float().numpy(), dy.float().numpy(), coef.float().numpy()
    assert hip.linear_projection_supported(T, in_f, out_f, k)
    xg, dyg, cg = x.cuda(), dy.cuda(), coef.cuda()
    z = hip.linear_project(xg, k, out_f, seed, coef=cg)
    noise = oracle.noise_2d(in_f, k, seed).astype(np.float64)          # noise[i, m] = noise(PRIME*i + m)
    want_z = xn.astype(np.float64) @ noise
    pieces = hip.projection_unpack(z, in_f, out_f, k)                  # the state holds z twice and the coefficients once
    assert pieces["z"].shape == (T, k) and rel_l2(cpu(pieces["z"]), want_z) < 5e-3  # one bf16 rounding of z
    assert torch.equal(pieces["z_t"], pieces["z"].t()) and torch.equal(pieces["coef_t"], cg.t())
    assert hip.projection_unpack(hip.linear_project(xg, k, out_f, seed), in_f, out_f, k)["coef_t"] is None
    bias = torch.randn(out_f).bfloat16()
    y = hip.linear_fwd_projected(z, cg, in_f, seed, bias=bias.cuda())
    want_y = oracle.linear_fwd(xn, cn, in_f, out_f, seed, bias=bias.float().numpy())
    assert y.shape == (T, out_f) and rel_l2(cpu(y), want_y) < BF16_TOL
    dc = hip.linear_bwd_dcoef_projected(dyg, z, k, in_f, seed)
    _, want_dc, _ = oracle.linear_bwd(xn, dyn, cn, in_f, out_f, seed)
    assert dc.shape == (out_f, k) and rel_l2(cpu(dc), want_dc) < BF16_TOL
    # the one-call entry points do the same arithmetic: equal up to the order of the fp32 atomics
    y1 = hip.linear_fwd(xg, cg, in_f, out_f, in_f, 1, seed, bias=bias.cuda(), algo=3)
    assert torch.equal(y1, y)
    dc1, _ = hip.linear_bwd_dcoef(dyg, xg, k, out_f, in_f, out_f, in_f, 1, seed, algo=3)
    assert rel_l2(cpu(dc1), cpu(dc)) < 1e-5


@pytest.mark.parametrize("T,in_f,out_f,k,seed", BWD_SHAPES + [(8192, 768, 3072, 256, 0), (1000, 200, 328, 72, 5), (300, 128, 256, 512, 2)])
def test_project_fwd_in_one_call(hip, T, in_f, out_f, k, seed):
    """Projection and forward product in one call (one launch for k <= 256: the multiplying blocks wait for the tags of the
    projecting blocks) against the two separate calls: same bits in y and in every piece of the state, on a state buffer
    that held other bytes before and again on the buffer the first call wrote."""
    print(f"case project+fwd T={T} in={in_f} out={out_f} k={k}", flush=True)
    x, _, coef = _inputs(T, in_f, out_f, k, True, torch.bfloat16, seed)
    xg, cg = x.cuda(), coef.cuda()
    bias = torch.randn(out_f).bfloat16().cuda()
    want_state = hip.linear_project(xg, k, out_f, seed, coef=cg)
    want_y = hip.linear_fwd_projected(want_state, cg, in_f, seed, bias=bias)
    want = hip.projection_unpack(want_state, in_f, out_f, k)
    for round_ in range(3):
        y, state = hip.linear_project_fwd(xg, cg, seed, bias=bias)
        got = hip.projection_unpack(state, in_f, out_f, k)
        assert torch.equal(y, want_y), f"y differs in round {round_}"
        for name in ("z", "z_t", "coef_t"):
            assert torch.equal(got[name], want[name]), f"{name} differs in round {round_}"
        assert int(state.view(-1)[:8].view(torch.int32)[1]) == 0, "a block gave up waiting for the projection"
    y_nb, _ = hip.linear_project_fwd(xg, cg, seed)
    assert torch.equal(y_nb, hip.linear_fwd_projected(want_state, cg, in_f, seed))


def test_a_wait_that_gives_up_is_loud(hip):
    """Only the consumer blocks of the one-launch forward run, on a tag nobody publishes and with a wait of 32 polls: every
    block gives up, every kernel ends normally, y is NaN throughout (never a product of whatever lay in memory), the state says
    so, the host-side watch raises and switches the library to separate launches; with the switch back on, the next one-launch
    call on the same state gives the bits of the two separate calls again.  bf16 (projection state) and fp32 small k (workspace)."""
    from randumb_amd import _lib

    print("case bounded wait gives up: bf16", flush=True)
    T, in_f, out_f, k, seed = 1000, 264, 520, 136, 4
    x, _, coef = _inputs(T, in_f, out_f, k, True, torch.bfloat16, seed)
    xg, cg = x.cuda(), coef.cuda()
    hip.sync_check()   # whatever earlier tests left is looked at here
    want_y, state = hip.linear_project_fwd(xg, cg, seed)
    y = torch.zeros_like(want_y)
    hip.selftest_sync_giveup(y, state, cg, in_f, seed, polls=32)
    torch.cuda.synchronize()
    assert bool(torch.isnan(y.float()).all()), "a block that gave up stored something other than NaN"
    assert int(state.view(-1)[:8].view(torch.int32)[1]) == 2
    with pytest.raises(_lib.RandumbHipError, match="gave up"):
        hip.sync_check()
    assert hip.set_one_launch(1) == 0, "the watch did not switch the one-launch forms off"
    hip.sync_check()   # nothing new: no error
    y2, state2 = hip.linear_project_fwd(xg, cg, seed)
    assert torch.equal(y2, want_y) and int(state2.view(-1)[:8].view(torch.int32)[1]) == 0
    want_state = hip.linear_project(xg, k, out_f, seed, coef=cg)
    assert torch.equal(hip.linear_fwd_projected(want_state, cg, in_f, seed), want_y)
    # separate launches give the same bits
    assert hip.set_one_launch(0) == 1
    try:
        y3, _ = hip.linear_project_fwd(xg, cg, seed)
        assert torch.equal(y3, want_y)
    finally:
        hip.set_one_launch(1)

    print("case bounded wait gives up: fp32 small k", flush=True)
    T, in_f, out_f, k, seed = 37, 1000, 520, 16, 9
    x, _, coef = _inputs(T, in_f, out_f, k, True, torch.float32, seed)
    xg, cg = x.cuda(), coef.cuda()
    want = hip.linear_fwd(xg, cg, in_f, out_f, in_f, 1, seed)
    d = hip._desc(T, in_f, out_f, cg, in_f, 1, seed, torch.float32, 0)
    import ctypes
    ws = torch.zeros(int(_lib.load().rdb_linear_workspace_bytes(0, ctypes.byref(d))), dtype=torch.uint8, device="cuda")
    y = torch.zeros(T, out_f, device="cuda")
    hip.selftest_sync_giveup(y, ws, cg, in_f, seed, polls=32)
    torch.cuda.synchronize()
    assert bool(torch.isnan(y).all())
    with pytest.raises(_lib.RandumbHipError, match="gave up"):
        hip.sync_check()
    hip.set_one_launch(0)
    try:
        two = hip.linear_fwd(xg, cg, in_f, out_f, in_f, 1, seed)
    finally:
        hip.set_one_launch(1)
    assert torch.equal(two, want) and torch.equal(hip.linear_fwd(xg, cg, in_f, out_f, in_f, 1, seed), want)


def test_projected_calls_take_leading_dimensions(hip):
    """x and dy as column slices of wider matrices (row stride larger than the row): the projected calls read them in place and
    give the bits they give on contiguous copies."""
    print("case projected calls on strided activations", flush=True)
    T, in_f, out_f, k, seed = 700, 264, 520, 136, 4
    g = torch.Generator().manual_seed(8)
    xw = torch.randn(T, in_f + 40, generator=g).bfloat16().cuda()
    dyw = torch.randn(T, out_f + 24, generator=g).bfloat16().cuda()
    C = (torch.randn(out_f, k, generator=g) * 0.05).bfloat16().cuda()
    x, dy = xw[:, 16:16 + in_f], dyw[:, 8:8 + out_f]          # 16-byte aligned starts, strides in_f + 40 and out_f + 24
    assert x.stride(0) == in_f + 40 and dy.stride(0) == out_f + 24
    y, state = hip.linear_project_fwd(x, C, seed)
    dx, dC = hip.linear_bwd_projected(dy, state, C, in_f, seed)
    y_c, state_c = hip.linear_project_fwd(x.contiguous(), C, seed)
    dx_c, dC_c = hip.linear_bwd_projected(dy.contiguous(), state_c, C, in_f, seed)
    assert torch.equal(y, y_c) and torch.equal(dx, dx_c) and torch.equal(dC, dC_c)
    # the separate coefficient gradient adds its token ranges with fp32 atomics: equal up to their order
    assert rel_l2(cpu(hip.linear_bwd_dcoef_projected(dy, state, k, in_f, seed)), cpu(dC_c)) < 1e-5


@pytest.mark.parametrize("T,in_f,out_f,k,seed", BWD_SHAPES)
def test_linear_bwd_projected_one_call(hip, oracle, T, in_f, out_f, k, seed):
    """dx and dcoef from one call (two launches, dcoef blocks and dx blocks side by side) against the oracle and against
    the separate entry points."""
    print(f"case bwd projected T={T} in={in_f} out={out_f} k={k}", flush=True)
    x, dy, coef = _inputs(T, in_f, out_f, k, True, torch.bfloat16, seed)
    want_dx, want_dc, _ = oracle.linear_bwd(x.float().numpy(), dy.float().numpy(), coef.float().numpy(), in_f, out_f, seed)
    dyc, cc = dy.cuda(), coef.cuda()
    z_plain = hip.linear_project(x.cuda(), k, out_f, seed)            # without the transposed coefficients: dy.C reads C through LDS
    z = hip.linear_project(x.cuda(), k, out_f, seed, coef=cc)          # with them: dy.C takes them straight into registers
    dx_sep = hip.linear_bwd_dx(dyc, cc, in_f, out_f, in_f, 1, seed, algo=3)
    dc_sep = hip.linear_bwd_dcoef_projected(dyc, z, k, in_f, seed)
    dx_plain, dc_plain = hip.linear_bwd_projected(dyc, z_plain, cc, in_f, seed)
    assert torch.equal(dx_plain, dx_sep) and rel_l2(cpu(dc_plain), want_dc) < BF16_TOL
    for ordered in (True, False):   # partial sums added in order (bigger workspace) / combined with atomics
        runs = []
        for _ in range(2):   # the second call finds dcoef's buffer dirty in the allocator: it must be overwritten by the call
            dx, dc = hip.linear_bwd_projected(dyc, z, cc, in_f, seed, ordered_sums=ordered)
            assert dx.shape == (T, in_f) and rel_l2(cpu(dx), want_dx) < BF16_TOL
            assert dc.shape == (out_f, k) and rel_l2(cpu(dc), want_dc) < BF16_TOL
            runs.append(dc)
        assert torch.equal(dx, dx_sep)
        assert rel_l2(cpu(dc), cpu(dc_sep)) < 1e-5
        if ordered:
            assert torch.equal(runs[0], runs[1])   # no atomics on this path: the same bits every time


def test_projected_form_rejects_what_it_cannot_do(hip):
    from randumb_amd._lib import RandumbHipError

    assert not hip.linear_projection_supported(64, 100, 32, 16)      # in_f not a multiple of 8
    x = torch.randn(64, 100, device="cuda").bfloat16()
    with pytest.raises(RandumbHipError):
        hip.linear_project(x, 16, 32, 0)
    with pytest.raises(ValueError):                                    # not a projection state
        hip.linear_fwd_projected(torch.randn(64, 16, device="cuda").bfloat16(), torch.randn(32, 16, device="cuda").bfloat16(), 96, 0)
    z = hip.linear_project(torch.randn(64, 96, device="cuda").bfloat16(), 16, 32, 0)
    c32 = torch.randn(32, 16, device="cuda")                          # fp32 coefficients: not in the projected forward
    with pytest.raises(RandumbHipError):
        hip.linear_fwd_projected(z, c32, 96, 0)


def test_factored_dx_needs_what_it_says(hip):
    from randumb_amd._lib import RandumbHipError, RDB_ALGO_FACTORED

    dy = torch.randn(64, 48, device="cuda").bfloat16()
    c = torch.randn(16, device="cuda").bfloat16()          # vector-coef has no factored form
    with pytest.raises(RandumbHipError):
        hip.linear_bwd_dx(dy, c, 40, 48, 40, 1, 0, algo=RDB_ALGO_FACTORED)
    C = torch.randn(48, 16, device="cuda").bfloat16()
    sb = torch.tensor([0.1], device="cuda").bfloat16()      # the random-bias term rides on top of the factored input gradient
    assert hip.linear_bwd_dx(dy, C, 40, 48, 40, 1, 0, scale_bias=sb, algo=RDB_ALGO_FACTORED).shape == (64, 40)
    assert hip.linear_bwd_dx(dy, C, 40, 48, 40, 1, 0, scale_bias=sb).shape == (64, 40)
    x = torch.randn(64, 40, device="cuda").bfloat16()
    with pytest.raises(RandumbHipError):
        hip.linear_fwd(x, c, 40, 48, 40, 1, 0, algo=RDB_ALGO_FACTORED)
    with pytest.raises(RandumbHipError):
        hip.linear_fwd(x, C, 40, 48, 40, 1, 0, scale_bias=sb, algo=RDB_ALGO_FACTORED)
    with pytest.raises(RandumbHipError):
        hip.linear_bwd_dcoef(dy, x, 16, 0, 40, 48, 40, 1, 0, algo=RDB_ALGO_FACTORED)
    with pytest.raises(RandumbHipError):
        hip.linear_bwd_dcoef(dy, x, 16, 48, 40, 48, 40, 1, 0, want_scale_bias_grad=True, algo=RDB_ALGO_FACTORED)


@pytest.mark.parametrize("T,in_f,out_f,k", [
    (2048, 768, 3072, 256),
    (200, 72, 136, 40),
    (1024, 3072, 768, 256),   # in_f too long for a weight strip on chip: factored forward + the random-bias share added on top
    (512, 1024, 1024, 512),   # k > 256 and the factored form not the cheaper one in flops: still the one that runs
    (4000, 1032, 1048, 64),   # enough tiles of 512 tokens x 64 features for the eight-wave random-bias kernel in both directions, ragged against both
])
def test_default_layer_fast_path_with_scale_bias(hip, oracle, T, in_f, out_f, k):
    """The reference's default layer starts from zero coefficients and a fused random bias (SillyLayers.py:122-133, 218-221):
    W = C.N + s.noise1d.  Forward, input gradient (factored share + hashed random-bias share), coefficient gradient and the
    gradient of s through the entry points AUTO picks, against the oracle, with s != 0 and C != 0 and with C = 0."""
    print(f"case scale_bias fast path T={T} in={in_f} out={out_f} k={k}", flush=True)
    x, dy, coef = _inputs(T, in_f, out_f, k, True, torch.bfloat16, 21)
    sbv = 0.0625     # exact in bf16; the weight's random share then has the size of the low-rank share
    sb = torch.tensor([sbv]).bfloat16()
    for c in (coef, torch.zeros_like(coef)):
        xn, dyn, cn = x.float().numpy(), dy.float().numpy(), c.float().numpy()
        want_y = oracle.linear_fwd(xn, cn, in_f, out_f, 9, scale_bias=sbv)
        want_dx, want_dc, dW = oracle.linear_bwd(xn, dyn, cn, in_f, out_f, 9, scale_bias=sbv)
        want_ds = float(oracle.scale_bias_bwd(dW.astype(np.float32), 9)[0])
        xg, dyg, cg, sg = x.cuda(), dy.cuda(), c.cuda(), sb.cuda()
        y = hip.linear_fwd(xg, cg, in_f, out_f, in_f, 1, 9, scale_bias=sg)
        dx = hip.linear_bwd_dx(dyg, cg, in_f, out_f, in_f, 1, 9, scale_bias=sg)
        dc, ds = hip.linear_bwd_dcoef(dyg, xg, k, out_f, in_f, out_f, in_f, 1, 9, want_scale_bias_grad=True)
        assert rel_l2(cpu(y), want_y) < BF16_TOL
        assert rel_l2(cpu(dx), want_dx) < BF16_TOL
        assert rel_l2(cpu(dc), want_dc) < BF16_TOL
        assert abs(float(ds) - want_ds) < BF16_TOL * max(abs(want_ds), float(np.linalg.norm(dW)))
        # input gradient and the gradient of s from one pass over dy.R (what the layer's backward pass calls): the same dx bit
        # for bit, d s = <dy.R, x> against the oracle and the same bits run to run; the coefficient gradient then needs no dW
        both = hip.linear_bwd_dx_dscale(dyg, xg, cg, in_f, out_f, 9, sg)
        assert both is not None and torch.equal(both[0], dx)
        assert abs(float(both[1]) - want_ds) < BF16_TOL * max(abs(want_ds), float(np.linalg.norm(dW)))
        # (the dW-tile kernel above rounds dW to bf16 before the contraction, this one reduces fp32 sums: it is the closer one)
        assert torch.equal(hip.linear_bwd_dx_dscale(dyg, xg, cg, in_f, out_f, 9, sg)[1], both[1])
        # the random-bias share as calls of its own on top of the projected entry points (what the layer runs: z = x.N^T is formed
        # once, by the forward pass): the same kernels in the same order as inside rdb_linear_fwd / rdb_linear_bwd_dx_dscale
        if hip.linear_projection_supported(T, in_f, out_f, k):
            y2, state = hip.linear_project_fwd(xg, cg, 9, None)
            hip.linear_rbias_fwd_(y2, xg, sg, in_f, out_f, 9)
            assert rel_l2(cpu(y2), want_y) < BF16_TOL
            dx2, dc2 = hip.linear_bwd_projected(dyg, state, cg, in_f, 9)
            ds2 = hip.linear_rbias_bwd_(dx2, dyg, xg, sg, in_f, out_f, 9, want_scale_bias_grad=True)
            assert rel_l2(cpu(dx2), want_dx) < BF16_TOL and rel_l2(cpu(dc2), want_dc) < BF16_TOL
            assert torch.equal(ds2, both[1]), "the gradient of the scale does not depend on what dx held"
            dx3, _ = hip.linear_bwd_projected(dyg, state, cg, in_f, 9)
            assert hip.linear_rbias_bwd_(dx3, dyg, None, sg, in_f, out_f, 9) is None and torch.equal(dx3, dx2)
        dc_only, none = hip.linear_bwd_dcoef(dyg, xg, k, out_f, in_f, out_f, in_f, 1, 9, want_scale_bias_grad=False)
        assert none is None and rel_l2(cpu(dc_only), want_dc) < BF16_TOL
        # the same input gradient from the general kernel that forms the weight block by block
        from randumb_amd._lib import RDB_ALGO_TILE
        if T <= 256:
            dx_t = hip.linear_bwd_dx(dyg, cg, in_f, out_f, in_f, 1, 9, scale_bias=sg, algo=RDB_ALGO_TILE)
            assert rel_l2(cpu(dx), cpu(dx_t)) < 1e-2


def test_projected_path_random_shapes(hip, oracle):
    """Twenty random layer shapes (multiples of 8, ragged against every tile size) through the projected entry points, with
    and without bias, with the workspace for ordered sums and with the smaller one."""
    rng = np.random.default_rng(2024)
    for case in range(20):
        T = int(rng.integers(1, 90)) * 8 - int(rng.integers(0, 8))          # tokens need not be a multiple of anything
        in_f, out_f, k = (int(rng.integers(1, 66)) * 8 for _ in range(3))
        seed = int(rng.integers(0, 2**32))
        print(f"case random projected {case}: T={T} in={in_f} out={out_f} k={k} seed={seed}", flush=True)
        x, dy, coef = _inputs(T, in_f, out_f, k, True, torch.bfloat16, case)
        xn, dyn, cn = x.float().numpy(), dy.float().numpy(), coef.float().numpy()
        xg, dyg, cg = x.cuda(), dy.cuda(), coef.cuda()
        bias = torch.randn(out_f).bfloat16() if case % 2 == 0 else None
        z = hip.linear_project(xg, k, out_f, seed)
        y = hip.linear_fwd_projected(z, cg, in_f, seed, bias=None if bias is None else bias.cuda())
        dx, dc = hip.linear_bwd_projected(dyg, z, cg, in_f, seed, ordered_sums=case % 3 != 0)
        want_dx, want_dc, _ = oracle.linear_bwd(xn, dyn, cn, in_f, out_f, seed)
        want_y = oracle.linear_fwd(xn, cn, in_f, out_f, seed, bias=None if bias is None else bias.float().numpy())
        assert rel_l2(cpu(y), want_y) < BF16_TOL, case
        assert rel_l2(cpu(dx), want_dx) < BF16_TOL, case
        assert rel_l2(cpu(dc), want_dc) < BF16_TOL, case
