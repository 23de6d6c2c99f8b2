"""GPU parity at the benchmark configurations' real shapes.

The small configuration (MNIST-shaped MLP) is covered in test_gpu_surface.py.  Here: the headline layer at full size, the
small-k fp32 regime, the LLM-sized layer and the GPT-2 layer shapes with seeds 0..47.  At sizes where the CPU oracle would
take minutes, the comparison runs on slices that the algorithm makes independent (a token's y and dx depend on that token
only; in matrix-coef form a weight row depends on its coefficient row only) and on size-independent identities
(adjoint: <dC, C'> = <dy, x W(C')^T>).  Tolerances (relative L2): fp32 1e-5, bf16 2e-2.
"""
import math

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


def cpu(t):
    return t.detach().float().cpu().numpy()


@pytest.fixture(scope="module")
def hip():
    assert torch.cuda.is_available(), "these tests need the MI355X"
    from randumb_amd import hip as h

    return h


@pytest.fixture(scope="module")
def ra():
    assert torch.cuda.is_available(), "these tests need the MI355X"
    import randumb_amd

    return randumb_amd


def _layer_inputs(T, in_f, out_f, k, std, seed, dtype):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(T, in_f, generator=g).to(dtype)
    dy = torch.randn(T, out_f, generator=g).to(dtype)
    C = (torch.randn(out_f, k, generator=g) * (3.0 * std * std / k) ** 0.5).to(dtype)
    return x, dy, C


def _check_bf16_layer_on_slices(hip, oracle, T, in_f, out_f, k, std, seed, n_tok=96, n_out=192):
    """Forward and backward of one matrix-coef bf16 layer at full size; oracle on a token slice and an output-row slice."""
    x, dy, C = _layer_inputs(T, in_f, out_f, k, std, seed, torch.bfloat16)
    rng = np.random.default_rng(seed)
    tok = np.sort(rng.choice(T, size=min(n_tok, T), replace=False))
    osel = np.sort(rng.choice(out_f, size=min(n_out, out_f), replace=False))
    # dy restricted to the chosen output rows, so that dx needs only those rows of W
    dy_s = torch.zeros_like(dy)
    dy_s[:, osel] = dy[:, osel]
    xg, dyg, dysg, Cg = x.cuda(), dy.cuda(), dy_s.cuda(), C.cuda()

    z = hip.linear_project(xg, k, out_f, seed)
    y = hip.linear_fwd_projected(z, Cg, in_f, seed)
    dx_s, _ = hip.linear_bwd_projected(dysg, z, Cg, in_f, seed)
    dx, dC = hip.linear_bwd_projected(dyg, z, Cg, in_f, seed)
    torch.cuda.synchronize()

    xn, Cn = x.float().numpy(), C.float().numpy()
    # forward: chosen tokens x chosen output rows against materialise-then-matmul on the oracle
    want_y = oracle.linear_fwd(xn[tok], Cn[osel], in_f, len(osel), seed)
    assert rel_l2(cpu(y)[np.ix_(tok, osel)], want_y) < BF16_TOL
    # dx for the chosen tokens, dy restricted to the chosen rows
    want_dx, _, _ = oracle.linear_bwd(xn[tok], dy.float().numpy()[np.ix_(tok, osel)], Cn[osel], in_f, len(osel), seed)
    assert rel_l2(cpu(dx_s)[tok], want_dx) < BF16_TOL
    # dC rows of the chosen outputs over ALL tokens: dC[o, :] = sum_t dy[t, o] * (x[t] . N^T), noise from the oracle
    noise = oracle.noise_2d(in_f, k, seed).astype(np.float64)
    zz = xn.astype(np.float64) @ noise
    want_dC = dy.float().numpy()[:, osel].astype(np.float64).T @ zz
    assert rel_l2(cpu(dC)[osel], want_dC) < BF16_TOL
    # full-size identities: dx is linear in dy; <dC, C'> = <dy, x W(C')^T> for another coefficient matrix C'
    dx_rest, _ = hip.linear_bwd_projected((dyg - dysg), z, Cg, in_f, seed)
    assert rel_l2(cpu(dx_s) + cpu(dx_rest), cpu(dx)) < BF16_TOL
    # <dC, C'> = <dy, x W(C')^T> for another coefficient matrix C'.  With a random C' both sides are the inner product of
    # nearly orthogonal vectors (|.| ~ norms / sqrt(N)) and any tolerance in terms of norms is vacuous, so C' is taken along
    # dC itself: both sides are then ~ |dC| |C'|, and a wrong scale, sign or a dropped token range of dC shows.
    Cp = (dC / dC.abs().max() * 0.02).bfloat16()
    yp = hip.linear_fwd_projected(z, Cp, in_f, seed)
    lhs = float((dC.double() * Cp.double()).sum())
    rhs = float((dyg.double() * yp.double()).sum())
    assert lhs > 0.5 * float(dC.double().norm() * Cp.double().norm())       # the probe is along dC
    assert abs(lhs - rhs) < BF16_TOL * abs(lhs), (lhs, rhs)
    return y, dx, dC


def test_headline_layer_full_size(hip, oracle):
    """768 -> 3072, k = 256, 8192 tokens, bf16, C ~ N(0, 3*0.02^2/k), seed 0: the configuration the benchmark times."""
    print("case config: headline layer 768->3072 k=256 T=8192", flush=True)
    y, dx, dC = _check_bf16_layer_on_slices(hip, oracle, 8192, 768, 3072, 256, 0.02, 0)
    assert y.shape == (8192, 3072) and dx.shape == (8192, 768) and dC.shape == (3072, 256)


def test_llm_sized_layer(hip, oracle):
    """4096 -> 14336, k = 1024, 4096 tokens, bf16, std = 1/sqrt(4096): W (58.7 M elements) is never written."""
    print("case config: LLM-sized layer 4096->14336 k=1024 T=4096", flush=True)
    y, dx, dC = _check_bf16_layer_on_slices(hip, oracle, 4096, 4096, 14336, 1024, 1.0 / 64.0, 3, n_tok=64, n_out=128)
    assert y.shape == (4096, 14336) and dx.shape == (4096, 4096) and dC.shape == (14336, 1024)


@pytest.mark.parametrize("T,in_f,out_f,k,std", [(8192, 768, 3072, 256, 0.02), (256, 4096, 1024, 1024, 1.0 / 64.0)])
def test_projected_form_against_the_kernels_that_form_the_weight(hip, T, in_f, out_f, k, std):
    """The factored products round z = x.N^T and t = dy.C to bf16 where the prescribed data flow rounds W = N.C to bf16 once
    (RandumbTensor.py:892).  The two must stay close: y, dx and dC of the projected entry points against the kernels that do
    form weight (and weight-gradient) tiles on chip, at the headline shape and at the k = 1024 layer's width."""
    print(f"case projected vs W-forming T={T} in={in_f} out={out_f} k={k}", flush=True)
    from randumb_amd._lib import RDB_ALGO_STRIP, RDB_ALGO_TILE

    x, dy, C = _layer_inputs(T, in_f, out_f, k, std, 11, torch.bfloat16)
    xg, dyg, Cg = x.cuda(), dy.cuda(), C.cuda()
    z = hip.linear_project(xg, k, out_f, 11, coef=Cg)
    y = hip.linear_fwd_projected(z, Cg, in_f, 11)
    dx, dC = hip.linear_bwd_projected(dyg, z, Cg, in_f, 11)
    algo = RDB_ALGO_STRIP if k <= 256 else RDB_ALGO_TILE
    y_w = hip.linear_fwd(xg, Cg, in_f, out_f, in_f, 1, 11, algo=algo)
    dx_w = hip.linear_bwd_dx(dyg, Cg, in_f, out_f, in_f, 1, 11, algo=algo)
    dC_w, _ = hip.linear_bwd_dcoef(dyg, xg, k, out_f, in_f, out_f, in_f, 1, 11, algo=algo)
    assert rel_l2(cpu(y), cpu(y_w)) < 1e-2
    assert rel_l2(cpu(dx), cpu(dx_w)) < 1e-2
    assert rel_l2(cpu(dC), cpu(dC_w)) < 1e-2


def test_more_tokens_than_one_launch_addresses(hip, oracle):
    """65536 tokens through 4096 -> 14336 (k = 256): dy and y hold 2^29.8 elements, more than one launch addresses, so the
    projected entry points run the layer in 4 chunks of 16384 tokens.  y and dx on tokens from every chunk (and both sides of
    every chunk boundary) against the oracle; dC rows against dy^T.(x.N^T) over ALL tokens in fp64 with the oracle's noise;
    dC the same bits on a second run (the chunks' sums are added in chunk order)."""
    print("case config: 65536 tokens x 4096->14336 k=256, chunked", flush=True)
    T, in_f, out_f, k, seed = 65536, 4096, 14336, 256, 5
    assert hip.linear_projection_supported(T, in_f, out_f, k)
    g = torch.Generator(device="cuda").manual_seed(3)
    x = torch.randn(T, in_f, generator=g, device="cuda", dtype=torch.float32).bfloat16()
    C = (torch.randn(out_f, k, generator=g, device="cuda") * (3.0 / k) ** 0.5 / 64.0).bfloat16()
    osel = np.sort(np.random.default_rng(0).choice(out_f, size=96, replace=False))
    tok = np.array([0, 1, 16383, 16384, 16385, 32767, 32768, 40000, 49151, 49152, 65534, 65535])
    # dy non-zero on the chosen output rows only (dx then needs only those rows of W), but on every token
    dy = torch.zeros(T, out_f, device="cuda", dtype=torch.bfloat16)
    dy[:, torch.from_numpy(osel).cuda()] = torch.randn(T, len(osel), generator=g, device="cuda").bfloat16()
    state = hip.linear_project(x, k, out_f, seed, coef=C)
    y = hip.linear_fwd_projected(state, C, in_f, seed)
    dx, dC = hip.linear_bwd_projected(dy, state, C, in_f, seed)
    dx2, dC2 = hip.linear_bwd_projected(dy, state, C, in_f, seed)
    torch.cuda.synchronize()
    assert y.shape == (T, out_f) and dx.shape == (T, in_f) and dC.shape == (out_f, k)
    assert torch.equal(dC, dC2) and torch.equal(dx, dx2)
    xs, Cs = cpu(x[tok]), cpu(C)[osel]
    assert rel_l2(cpu(y[tok])[:, osel], oracle.linear_fwd(xs, Cs, in_f, len(osel), seed)) < BF16_TOL
    want_dx, _, _ = oracle.linear_bwd(xs, cpu(dy[tok])[:, osel], Cs, in_f, len(osel), seed)
    assert rel_l2(cpu(dx[tok]), want_dx) < BF16_TOL
    noise = torch.from_numpy(oracle.noise_2d(in_f, k, seed)).cuda().double()
    want_dC = dy[:, torch.from_numpy(osel).cuda()].double().t() @ (x.double() @ noise)
    assert rel_l2(cpu(dC)[osel], want_dC.cpu().numpy()) < BF16_TOL
    rest = np.setdiff1d(np.arange(out_f), osel)[:64]
    assert float(dC[torch.from_numpy(rest).cuda()].abs().max()) == 0.0   # rows whose dy is zero
    # projection and forward product in one call per chunk: the same y, and a state that gives the same backward pass
    del dx2, dC2
    y1, state1 = hip.linear_project_fwd(x, C, seed)
    assert torch.equal(y1, y)
    del y1
    dx1, dC1 = hip.linear_bwd_projected(dy, state1, C, in_f, seed)
    assert torch.equal(dx1, dx) and torch.equal(dC1, dC)


@pytest.mark.parametrize("batch", [1, 16, 256])
@pytest.mark.parametrize("matrix", [True, False])
def test_small_k_fp32_regime(hip, oracle, batch, matrix):
    """4096 -> 4096, k = 16, fp32, batch 1 / 16 / 256 (GEMV-like).  rel-L2 <= 1e-5 against the oracle."""
    print(f"case config: small-k fp32 4096->4096 k=16 batch={batch} matrix={matrix}", flush=True)
    in_f = out_f = 4096
    k, seed = 16, 11
    g = torch.Generator().manual_seed(batch)
    x = torch.randn(batch, in_f, generator=g)
    dy = torch.randn(batch, out_f, generator=g)
    C = torch.randn((out_f, k) if matrix else (k,), generator=g) * (3.0 / k) ** 0.5 / 64.0
    y = hip.linear_fwd(x.cuda(), C.cuda(), in_f, out_f, in_f, 1, seed)
    dx = hip.linear_bwd_dx(dy.cuda(), C.cuda(), in_f, out_f, in_f, 1, seed)
    dC, _ = hip.linear_bwd_dcoef(dy.cuda(), x.cuda(), k, out_f if matrix else 0, in_f, out_f, in_f, 1, seed)
    want_y = oracle.linear_fwd(x.numpy(), C.numpy(), in_f, out_f, seed)
    want_dx, want_dC, _ = oracle.linear_bwd(x.numpy(), dy.numpy(), C.numpy(), in_f, out_f, seed)
    assert rel_l2(cpu(y), want_y) < F32_TOL
    assert rel_l2(cpu(dx), want_dx) < F32_TOL
    assert rel_l2(cpu(dC), want_dC) < F32_TOL
    if matrix:
        # AUTO takes the factored small-k kernels here; the kernels that form W tiles must agree, and so must a bias
        from randumb_amd._lib import RDB_ALGO_FACTORED, RDB_ALGO_TILE

        bias = torch.randn(out_f, generator=g)
        for algo in (RDB_ALGO_FACTORED, RDB_ALGO_TILE):
            yb = hip.linear_fwd(x.cuda(), C.cuda(), in_f, out_f, in_f, 1, seed, bias=bias.cuda(), algo=algo)
            assert rel_l2(cpu(yb), want_y + bias.numpy()) < F32_TOL, algo
            assert rel_l2(cpu(hip.linear_bwd_dx(dy.cuda(), C.cuda(), in_f, out_f, in_f, 1, seed, algo=algo)), want_dx) < F32_TOL, algo
            assert rel_l2(cpu(hip.linear_bwd_dcoef(dy.cuda(), x.cuda(), k, out_f, in_f, out_f, in_f, 1, seed, algo=algo)[0]), want_dC) < F32_TOL
        y2 = hip.linear_fwd(x.cuda(), C.cuda(), in_f, out_f, in_f, 1, seed, algo=RDB_ALGO_FACTORED)
        assert torch.equal(y2, hip.linear_fwd(x.cuda(), C.cuda(), in_f, out_f, in_f, 1, seed, algo=RDB_ALGO_FACTORED))  # reproducible


def test_small_k_fp32_long_contraction_runs_in_two_launches(hip, oracle):
    """More than 8192 input features: an expanding block would wait for more tags than a wave has lanes, so the contraction and
    the expansion run as two launches; same arithmetic, same tolerance."""
    from randumb_amd._lib import RDB_ALGO_FACTORED

    print("case small-k long contraction", flush=True)
    T, in_f, out_f, k, seed = 3, 8448, 64, 8, 21
    g = torch.Generator().manual_seed(6)
    x, dy = torch.randn(T, in_f, generator=g), torch.randn(T, out_f, generator=g)
    C = torch.randn(out_f, k, generator=g) * 0.1
    y = hip.linear_fwd(x.cuda(), C.cuda(), in_f, out_f, in_f, 1, seed, algo=RDB_ALGO_FACTORED)
    dx = hip.linear_bwd_dx(dy.cuda(), C.cuda(), in_f, out_f, in_f, 1, seed, algo=RDB_ALGO_FACTORED)
    want_dx, _, _ = oracle.linear_bwd(x.numpy(), dy.numpy(), C.numpy(), in_f, out_f, seed)
    assert rel_l2(cpu(y), oracle.linear_fwd(x.numpy(), C.numpy(), in_f, out_f, seed)) < F32_TOL
    assert rel_l2(cpu(dx), want_dx) < F32_TOL


def test_small_k_fp32_ragged_shapes(hip, oracle):
    """The fp32 small-k kernels on sizes that divide nothing: 5 tokens, 77 -> 130, k = 23, with bias."""
    from randumb_amd._lib import RDB_ALGO_FACTORED

    print("case small-k ragged", flush=True)
    T, in_f, out_f, k, seed = 5, 77, 130, 23, 9
    g = torch.Generator().manual_seed(4)
    x, dy = torch.randn(T, in_f, generator=g), torch.randn(T, out_f, generator=g)
    C, bias = torch.randn(out_f, k, generator=g) * 0.1, torch.randn(out_f, generator=g)
    y = hip.linear_fwd(x.cuda(), C.cuda(), in_f, out_f, in_f, 1, seed, bias=bias.cuda(), algo=RDB_ALGO_FACTORED)
    dx = hip.linear_bwd_dx(dy.cuda(), C.cuda(), in_f, out_f, in_f, 1, seed, algo=RDB_ALGO_FACTORED)
    dC, _ = hip.linear_bwd_dcoef(dy.cuda(), x.cuda(), k, out_f, in_f, out_f, in_f, 1, seed, algo=RDB_ALGO_FACTORED)
    want_dx, want_dC, _ = oracle.linear_bwd(x.numpy(), dy.numpy(), C.numpy(), in_f, out_f, seed)
    assert rel_l2(cpu(y), oracle.linear_fwd(x.numpy(), C.numpy(), in_f, out_f, seed, bias=bias.numpy())) < F32_TOL
    assert rel_l2(cpu(dx), want_dx) < F32_TOL and rel_l2(cpu(dC), want_dC) < F32_TOL


FEW_TOKEN_CASES = [(1, 2048, 1024, 256, False), (16, 1024, 2048, 256, True), (64, 1024, 768, 128, False), (33, 777, 555, 99, True),
                   (5, 8448, 512, 72, False), (80, 2048, 1536, 256, False)]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("T,in_f,out_f,k,with_bias", FEW_TOKEN_CASES)
def test_few_token_regime_up_to_k_256(hip, oracle, dtype, T, in_f, out_f, k, with_bias):
    """Up to 96 tokens (64 for the coefficient gradient) with k up to 256, both dtypes: the vector-ALU kernels compute in fp32 whatever the operands' dtype, so on
    bf16 operands y and dx carry one rounding to bf16 (rel-L2 about 1e-3; the bf16 matrix-core kernels, which also round z and
    t, are near 3e-3: the threshold between them shows which kernels ran) and the coefficient gradient, an fp32 result, meets
    the fp32 tolerance.  The last case contracts over
    more than 8192 features (two launches), the odd one divides nothing."""
    print(f"case few tokens: {dtype} T={T} {in_f}->{out_f} k={k} bias={with_bias}", flush=True)
    seed = 31
    g = torch.Generator().manual_seed(T + k)
    x = torch.randn(T, in_f, generator=g).to(dtype)
    dy = torch.randn(T, out_f, generator=g).to(dtype)
    C = (torch.randn(out_f, k, generator=g) * (3.0 / k) ** 0.5 / 32.0).to(dtype)
    bias = torch.randn(out_f, generator=g).to(dtype) if with_bias else None
    y = hip.linear_fwd(x.cuda(), C.cuda(), in_f, out_f, in_f, 1, seed, bias=None if bias is None else bias.cuda())
    dx = hip.linear_bwd_dx(dy.cuda(), C.cuda(), in_f, out_f, in_f, 1, seed)
    dC, _ = hip.linear_bwd_dcoef(dy.cuda(), x.cuda(), k, out_f, in_f, out_f, in_f, 1, seed)
    assert y.dtype == dtype and dx.dtype == dtype and dC.dtype == torch.float32
    xn, dyn, Cn = x.float().numpy(), dy.float().numpy(), C.float().numpy()
    want_y = oracle.linear_fwd(xn, Cn, in_f, out_f, seed, bias=None if bias is None else bias.float().numpy())
    want_dx, want_dC, _ = oracle.linear_bwd(xn, dyn, Cn, in_f, out_f, seed)
    # in bf16 the library takes these kernels for a direction whose contraction is long enough (1536 values) to leave the
    # matrix-core kernels behind (the coefficient gradient's is z = x.N^T, over in_f)
    tol_y = F32_TOL if dtype == torch.float32 else 2e-3 if in_f >= 1536 else BF16_TOL
    tol_dx = F32_TOL if dtype == torch.float32 else 2e-3 if out_f >= 1536 else BF16_TOL
    assert rel_l2(cpu(y), want_y) < tol_y
    assert rel_l2(cpu(dx), want_dx) < tol_dx
    # (sizes that are not multiples of 8 never take the bf16 matrix-core kernels: fp32-accurate either way)
    odd = in_f % 8 != 0 or out_f % 8 != 0 or k % 8 != 0
    assert rel_l2(cpu(dC), want_dC) < (F32_TOL if dtype == torch.float32 or (in_f >= 1536 and T <= 64) or odd else BF16_TOL)
    # bit for bit run to run (fixed summation order, no atomics), and as separate launches
    assert torch.equal(y, hip.linear_fwd(x.cuda(), C.cuda(), in_f, out_f, in_f, 1, seed, bias=None if bias is None else bias.cuda()))
    assert torch.equal(dC, hip.linear_bwd_dcoef(dy.cuda(), x.cuda(), k, out_f, in_f, out_f, in_f, 1, seed)[0])
    before = hip.set_one_launch(0)
    try:
        assert torch.equal(y, hip.linear_fwd(x.cuda(), C.cuda(), in_f, out_f, in_f, 1, seed, bias=None if bias is None else bias.cuda()))
        assert torch.equal(dx, hip.linear_bwd_dx(dy.cuda(), C.cuda(), in_f, out_f, in_f, 1, seed))
    finally:
        hip.set_one_launch(before)


def test_few_token_layer_through_the_surface(ra, hip, oracle):
    """A bf16 SillyLinear-shaped call with 8 tokens through ops.linear (autograd): takes the one-call entry points, not the
    projected form, and agrees with the oracle."""
    print("case few tokens through the surface", flush=True)
    from randumb_amd import ops

    T, in_f, out_f, k, seed = 8, 2048, 1536, 256, 5
    assert not hip.linear_projection_preferred(T, in_f, out_f, k, torch.bfloat16)
    assert hip.linear_projection_preferred(T, 1024, 1024, k, torch.bfloat16)   # short contractions: the matrix-core kernels
    assert hip.linear_projection_preferred(4096, in_f, out_f, k, torch.bfloat16)
    g = torch.Generator().manual_seed(2)
    x = torch.randn(T, in_f, generator=g).bfloat16().cuda().requires_grad_(True)
    C = (torch.randn(out_f, k, generator=g) * 0.01).bfloat16().cuda().requires_grad_(True)
    dy = torch.randn(T, out_f, generator=g).bfloat16().cuda()
    y = ops.linear(x, C, in_f, out_f, in_f, 1, seed, None, None)
    y.backward(dy)
    xn, dyn, Cn = cpu(x), cpu(dy), cpu(C)
    want_dx, want_dC, _ = oracle.linear_bwd(xn, dyn, Cn, in_f, out_f, seed)
    assert rel_l2(cpu(y), oracle.linear_fwd(xn, Cn, in_f, out_f, seed)) < 2e-3
    assert rel_l2(cpu(x.grad), want_dx) < 2e-3
    assert rel_l2(cpu(C.grad), want_dC) < 4e-3   # the gradient leaves in the coefficients' dtype


GPT2_SHAPES = [("qkv", 768, 2304), ("proj", 768, 768), ("fc", 768, 3072), ("mlp_proj", 3072, 768)]


def test_gpt2_layer_shapes_and_seeds(hip, oracle):
    """The four random-backed linears of a GPT-2 small block (k = 256, bf16), seeds 0..47 in layer order: every seed's noise
    bit-exact, and forward + backward of the two blocks at the ends (seeds 0..3 and 44..47) against the oracle on 256
    tokens; all 48 layers run at the full 8192 tokens and must satisfy the adjoint identity."""
    print("case config: GPT-2 small layer shapes, seeds 0..47", flush=True)
    k = 256
    for seed in range(48):
        got = hip.sq5_fill_2d(64, k, seed).cpu().numpy()
        assert np.array_equal(got.view(np.uint32), oracle.noise_2d(64, k, seed).view(np.uint32)), f"seed {seed}"
    for seed in range(48):
        name, in_f, out_f = GPT2_SHAPES[seed % 4]
        if seed < 4 or seed >= 44:
            x, dy, C = _layer_inputs(256, in_f, out_f, k, 0.02, seed, torch.bfloat16)
            z = hip.linear_project(x.cuda(), k, out_f, seed)
            y = hip.linear_fwd_projected(z, C.cuda(), in_f, seed)
            dx, dC = hip.linear_bwd_projected(dy.cuda(), z, C.cuda(), in_f, seed)
            xn, dyn, Cn = x.float().numpy(), dy.float().numpy(), C.float().numpy()
            want_dx, want_dC, _ = oracle.linear_bwd(xn, dyn, Cn, in_f, out_f, seed)
            assert rel_l2(cpu(y), oracle.linear_fwd(xn, Cn, in_f, out_f, seed)) < BF16_TOL, (name, seed)
            assert rel_l2(cpu(dx), want_dx) < BF16_TOL, (name, seed)
            assert rel_l2(cpu(dC), want_dC) < BF16_TOL, (name, seed)
        # full token count, every seed: <dC, C> = <dy, y> (y is linear in C) and <dx, x> = <dy, y> (y is linear in x).  dy is
        # taken along y (y plus noise of the same size), so that <dy, y> ~ |dy| |y| and the 2 % tolerance is relative to the
        # quantity compared; with an independent dy the inner products would be ~ norms / sqrt(N) and the check vacuous.
        x, dy, C = _layer_inputs(8192, in_f, out_f, k, 0.02, 100 + seed, torch.bfloat16)
        xg, Cg = x.cuda(), C.cuda()
        z = hip.linear_project(xg, k, out_f, seed, coef=Cg)
        y = hip.linear_fwd_projected(z, Cg, in_f, seed)
        dyg = (y.float() + dy.cuda().float() * y.float().std()).bfloat16()
        dx, dC = hip.linear_bwd_projected(dyg, z, Cg, in_f, seed)
        ref = float((dyg.double() * y.double()).sum())
        assert ref > 0.5 * float(dyg.double().norm() * y.double().norm()), (name, seed)
        assert abs(float((dC.double() * Cg.double()).sum()) - ref) < BF16_TOL * ref, (name, seed)
        assert abs(float((dx.double() * xg.double()).sum()) - ref) < BF16_TOL * ref, (name, seed)


def test_gpt2_small_full_model_starts_at_ln_vocab(ra):
    """The assembled 12-layer model of the step-time configuration (48 random-backed linears, k = 256, seeds 0..47, bf16,
    8 x 1024 random tokens): with the head's weights small the loss starts near ln(50304) = 10.8258, the sanity anchor
    the reference's trainer notes (modded-nanogpt/train_gpt2.py:241), and one backward pass leaves a finite, non-zero
    gradient on every one of the 48 coefficient matrices."""
    print("case config: GPT-2 small, 12 layers, full size", flush=True)
    from randumb_amd.gpt import RT_GPT, RT_GPTConfig

    torch.manual_seed(0)
    model = RT_GPT(RT_GPTConfig(int_dim_gen=ra.listgen([256] * 48), seed_gen=ra.stepgen(0, 1)))
    with torch.no_grad():
        model.lm_head.weight.mul_(0.05)          # logits ~ 0.03: the softmax is uniform up to second order
    model = model.to(torch.bfloat16).cuda()
    linears = [m for m in model.modules() if isinstance(m, ra.SillyLinear)]
    assert len(linears) == 48 and [m.weight.seed for m in linears] == list(range(48))
    g = torch.Generator().manual_seed(7)
    idx = torch.randint(0, 50304, (8, 1024), generator=g).cuda()
    tgt = torch.randint(0, 50304, (8, 1024), generator=g).cuda()
    loss = model(idx, tgt)
    assert torch.isfinite(loss) and abs(float(loss.detach()) - math.log(50304)) < 0.03 * math.log(50304), float(loss.detach())
    loss.backward()
    for i, m in enumerate(linears):
        gr = m.weight_coef.grad
        assert gr is not None and gr.shape == m.weight_coef.shape and bool(torch.isfinite(gr.float()).all()), i
        assert float(gr.float().abs().max()) > 0.0, i


def test_gpt_with_random_embedding_and_head(ra):
    """The reference's model makes the token embedding and the output head random-backed as well
    (modded-nanogpt/gpt_models.py:303, 310).  A small model built that way: the embedding draws the first seed, the head the
    last; the loss starts at ln(vocab) (head weights of standard deviation 0.02 on normalised activations); gradients reach
    the embedding's and the head's coefficients; the head gives the same logits through the fused kernels and through the
    tensor-subclass dispatch."""
    print("case config: GPT with random-backed embedding and head", flush=True)
    from randumb_amd.gpt import RT_GPT, RT_GPTConfig

    torch.manual_seed(0)
    cfg = RT_GPTConfig(int_dim_gen=ra.listgen([16] * 10), seed_gen=ra.stepgen(0, 1), vocab_size=384, n_layer=2, n_head=2, n_embd=64,
                       random_embedding_and_head=True)
    model = RT_GPT(cfg).to(torch.bfloat16).cuda()
    assert isinstance(model.wte, ra.SillyEmbedding) and model.wte.weight.seed == 0
    assert isinstance(model.lm_head, ra.SillyLinear) and model.lm_head.weight.seed == 9
    g = torch.Generator().manual_seed(3)
    idx = torch.randint(0, 384, (4, 128), generator=g).cuda()
    tgt = torch.randint(0, 384, (4, 128), generator=g).cuda()
    loss = model(idx, tgt)
    assert torch.isfinite(loss) and abs(float(loss.detach()) - math.log(384)) < 0.05 * math.log(384), float(loss.detach())
    loss.backward()
    for name, p in (("wte", model.wte.weight_coef), ("lm_head", model.lm_head.weight_coef)):
        assert p.grad is not None and bool(torch.isfinite(p.grad.float()).all()) and float(p.grad.float().abs().max()) > 0.0, name
    x = torch.randn(512, 64, generator=g).bfloat16().cuda()
    model.lm_head.fused = True
    y_fused = model.lm_head(x)
    model.lm_head.fused = False
    y_disp = model.lm_head(x)
    assert rel_l2(cpu(y_fused), cpu(y_disp)) < BF16_TOL


def _tiny_gpt(dtype, fused):
    from randumb_amd.SillyLayers import SillyLinear, listgen, stepgen
    from randumb_amd.gpt import RT_GPT, RT_GPTConfig

    torch.manual_seed(0)
    cfg = RT_GPTConfig(int_dim_gen=listgen([16] * 8), seed_gen=stepgen(0, 1), vocab_size=384, n_layer=2, n_head=2, n_embd=64)
    model = RT_GPT(cfg).to(dtype).cuda()
    for m in model.modules():
        if isinstance(m, SillyLinear):
            m.fused = fused
    return model


def test_gpt_block_wiring_matches_dispatch_path(hip, oracle):
    """A 2-layer GPT of random-backed linears (seeds 0..7 in qkv, proj, fc, mlp-proj order): the fused kernels and the
    materialise-then-matmul dispatch path give the same loss and coefficient gradients (fp32, tight), and the first block's
    qkv weight is the oracle's for seed 0."""
    print("case config: GPT wiring, 2 layers", flush=True)
    g = torch.Generator().manual_seed(5)
    idx = torch.randint(0, 384, (2, 48), generator=g).cuda()
    tgt = torch.randint(0, 384, (2, 48), generator=g).cuda()
    losses, grads = [], []
    for fused in (True, False):
        model = _tiny_gpt(torch.float32, fused)
        seeds = [m.seed[0] for m in model.modules() if hasattr(m, "weight_coef")]
        assert seeds == list(range(8))
        loss = model(idx, tgt)
        loss.backward()
        losses.append(float(loss.detach()))
        grads.append([cpu(m.weight_coef.grad) for m in model.modules() if hasattr(m, "weight_coef")])
    assert abs(losses[0] - losses[1]) < 1e-4 * abs(losses[1])
    for a, b in zip(*grads):
        assert rel_l2(a, b) < 1e-3
    qkv = model.h[0].attn.c_qkv
    W = oracle.materialize_fwd(cpu(qkv.weight_coef), (192, 64), (64, 1), 0, row_len=64)
    x = torch.randn(5, 64, generator=g)
    assert rel_l2(cpu(qkv(x.cuda())), x.numpy().astype(np.float64) @ W.astype(np.float64).T) < F32_TOL


def test_gpt_step_bf16(hip):
    """The same model in bf16 through the projected kernels: finite loss close to the fp32 one, a gradient for every coef."""
    print("case config: GPT wiring bf16 step", flush=True)
    g = torch.Generator().manual_seed(5)
    idx = torch.randint(0, 384, (2, 48), generator=g).cuda()
    tgt = torch.randint(0, 384, (2, 48), generator=g).cuda()
    ref = float(_tiny_gpt(torch.float32, True)(idx, tgt))
    model = _tiny_gpt(torch.bfloat16, True)
    loss = model(idx, tgt)
    loss.backward()
    assert abs(float(loss) - ref) < 2e-2 * abs(ref)
    for m in model.modules():
        if hasattr(m, "weight_coef"):
            gr = m.weight_coef.grad
            assert gr is not None and bool(torch.isfinite(gr).all()) and float(gr.float().abs().sum()) > 0
