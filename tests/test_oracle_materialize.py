"""Pins the oracle's materialise / gradient functions with facts the mathematics fixes.

None of these checks retypes the oracle's loop: each uses a special case that collapses to the
(already pinned) noise function, a brute-force dense product, or an algebraic identity
(linearity, adjointness, transposition) that a dropped term, wrong index or swapped operand breaks.
Reference: src/rten_cpp/RandumbTensor.py:235-290 (fwd), :304-359 (bwd), :399-420 (bias bwd),
:998-1108 (embedding).
"""
import numpy as np
import pytest


def rel_l2(a, b):
    a = np.asarray(a, dtype=np.float64)
    b = np.asarray(b, dtype=np.float64)
    return np.linalg.norm(a - b) / max(np.linalg.norm(b), 1e-30)


@pytest.mark.parametrize("P,Q,k,seed", [(3, 6, 18, 1337), (1, 37, 5, 0), (16, 16, 64, 47), (7, 5, 1, 9)])
def test_unit_vector_coef_gives_noise_column(oracle, P, Q, k, seed):
    noise = oracle.noise_2d_np(np.arange(P * Q), np.arange(k), seed)
    for j in {0, k // 2, k - 1}:
        c = np.zeros(k, dtype=np.float32)
        c[j] = 1.0
        W = oracle.materialize_fwd(c, (P, Q), (Q, 1), seed)
        assert np.array_equal(W.reshape(-1), noise[:, j])  # bit exact


def test_zero_coef_and_scale_bias(oracle):
    P, Q, k, seed = 5, 9, 12, 1337
    z = np.zeros(k, dtype=np.float32)
    assert not oracle.materialize_fwd(z, (P, Q), (Q, 1), seed).any()
    W = oracle.materialize_fwd(z, (P, Q), (Q, 1), seed, scale_bias=0.25)
    assert np.array_equal(W.reshape(-1), np.float32(0.25) * oracle.noise_1d(P * Q, seed))


def test_dense_bruteforce_and_fp32_order(oracle):
    rng = np.random.default_rng(0)
    P, Q, k, seed = 18, 18, 18, 1337  # the shape the reference's check_func uses (benchmark.py:134)
    c = rng.standard_normal(k).astype(np.float32)
    noise = oracle.noise_2d_np(np.arange(P * Q), np.arange(k), seed).astype(np.float64)
    want = (noise @ c.astype(np.float64)).reshape(P, Q)
    got = oracle.materialize_fwd(c, (P, Q), (Q, 1), seed)
    assert np.array_equal(got, want.astype(np.float32))
    got32 = oracle.materialize_fwd(c, (P, Q), (Q, 1), seed, acc_double=False)
    assert rel_l2(got32, want) < 1e-6
    assert rel_l2(oracle.materialize_fwd_np(c, (P, Q), (Q, 1), seed), want) < 1e-15


def test_linearity_in_coef(oracle):
    rng = np.random.default_rng(1)
    P, Q, k, seed = 8, 11, 32, 3
    a, b = rng.standard_normal((2, k)).astype(np.float32)
    Wa = oracle.materialize_fwd(a, (P, Q), (Q, 1), seed).astype(np.float64)
    Wb = oracle.materialize_fwd(b, (P, Q), (Q, 1), seed).astype(np.float64)
    Wab = oracle.materialize_fwd((2 * a - 3 * b).astype(np.float32), (P, Q), (Q, 1), seed)
    assert rel_l2(Wab, 2 * Wa - 3 * Wb) < 1e-6


def test_transposed_strides_and_1d_promotion(oracle):
    rng = np.random.default_rng(2)
    P, Q, k, seed = 6, 10, 16, 1337
    c = rng.standard_normal(k).astype(np.float32)
    W = oracle.materialize_fwd(c, (P, Q), (Q, 1), seed, scale_bias=0.5)
    Wt = oracle.materialize_fwd(c, (Q, P), (1, Q), seed, scale_bias=0.5)  # what aten.t() on the tensor yields
    assert np.array_equal(Wt, W.T)
    v1 = oracle.materialize_fwd(c, (Q,), (1,), seed)
    v2 = oracle.materialize_fwd(c, (1, Q), (0, 1), seed)
    assert np.array_equal(v1, v2.reshape(-1))
    assert np.array_equal(v1, W_first_row(oracle, c, Q, seed))


def W_first_row(oracle, c, Q, seed):
    return oracle.materialize_fwd(c, (1, Q), (Q, 1), seed).reshape(-1)


def test_matrix_coef_rows_are_vector_coef_tensors(oracle):
    """Row o of the matrix-coef form is a vector-coef tensor of shape (in,) with coef C[o, :]."""
    rng = np.random.default_rng(3)
    out_f, in_f, k, seed = 7, 13, 24, 47
    C = rng.standard_normal((out_f, k)).astype(np.float32)
    W = oracle.materialize_fwd(C, (out_f, in_f), (in_f, 1), seed, row_len=in_f)
    for o in range(out_f):
        row = oracle.materialize_fwd(C[o], (in_f,), (1,), seed)
        assert np.array_equal(W[o], row)
    # W = C @ N with N[m, i] = noise(i, m)
    N = oracle.noise_2d_np(np.arange(in_f), np.arange(k), seed).T.astype(np.float64)
    assert rel_l2(W, C.astype(np.float64) @ N) < 1e-7
    assert rel_l2(oracle.materialize_fwd_np(C, (out_f, in_f), (in_f, 1), seed, row_len=in_f),
                  C.astype(np.float64) @ N) < 1e-15
    Wt = oracle.materialize_fwd(C, (in_f, out_f), (1, in_f), seed, row_len=in_f)
    assert np.array_equal(Wt, W.T)


def test_bwd_unit_vector_and_ones(oracle):
    P, Q, k, seed = 4, 9, 20, 1337
    Nw = P * Q
    noise = oracle.noise_2d_np(np.arange(Nw), np.arange(k), seed)
    for n in (0, 17, Nw - 1):
        d = np.zeros(Nw, dtype=np.float32)
        d[n] = 1.0
        assert np.array_equal(oracle.materialize_bwd(d, k, seed), noise[n])
    ones = np.ones(Nw, dtype=np.float32)  # benchmark.py:377 uses dout = ones
    assert rel_l2(oracle.materialize_bwd(ones, k, seed), noise.astype(np.float64).sum(0)) < 1e-7


def test_bwd_is_the_adjoint_of_fwd(oracle):
    rng = np.random.default_rng(4)
    P, Q, k, seed = 12, 7, 33, 5
    c = rng.standard_normal(k).astype(np.float32)
    d = rng.standard_normal(P * Q).astype(np.float32)
    W = oracle.materialize_fwd(c, (P, Q), (Q, 1), seed).astype(np.float64).reshape(-1)
    dc = oracle.materialize_bwd(d, k, seed).astype(np.float64)
    assert abs(W @ d - c.astype(np.float64) @ dc) < 1e-5 * abs(W @ d)
    assert rel_l2(oracle.materialize_bwd_np(d, k, seed), dc) < 1e-6
    # matrix-coef form
    C = rng.standard_normal((P, k)).astype(np.float32)
    W2 = oracle.materialize_fwd(C, (P, Q), (Q, 1), seed, row_len=Q).astype(np.float64).reshape(-1)
    dC = oracle.materialize_bwd(d, k, seed, coef_rows=P).astype(np.float64)
    assert abs(W2 @ d - (C.astype(np.float64) * dC).sum()) < 1e-5 * abs(W2 @ d)
    assert rel_l2(oracle.materialize_bwd_np(d, k, seed, coef_rows=P), dC) < 1e-6
    for o in range(P):  # row o of dC is the vector-coef gradient of row o of dW
        assert np.array_equal(dC[o].astype(np.float32), oracle.materialize_bwd(d.reshape(P, Q)[o], k, seed))


def test_finite_difference_gradient(oracle):
    """d/dc <W(c), G> equals materialize_bwd(G) (central differences on the fp64 restatement)."""
    rng = np.random.default_rng(5)
    P, Q, k, seed = 3, 6, 18, 1337
    c = rng.standard_normal(k)
    G = rng.standard_normal(P * Q)
    f = lambda cc: float(oracle.materialize_fwd_np(cc, (P, Q), (Q, 1), seed).reshape(-1) @ G)
    g = np.array([(f(c + 1e-4 * e) - f(c - 1e-4 * e)) / 2e-4 for e in np.eye(k)])
    assert rel_l2(oracle.materialize_bwd(G, k, seed), g) < 1e-6


def test_scale_bias_bwd_closed_form(oracle):
    rng = np.random.default_rng(6)
    Nw, seed = 501, 77
    d = rng.standard_normal(Nw).astype(np.float32)
    want = d.astype(np.float64) @ oracle.noise_1d_np(np.arange(Nw, dtype=np.uint32), seed).astype(np.float64)
    assert abs(float(oracle.scale_bias_bwd(d, seed)[0]) - want) < 1e-6 * max(1.0, abs(want))


def test_embedding_is_a_row_gather(oracle):
    rng = np.random.default_rng(7)
    rows, rowsize, k, seed = 50, 24, 16, 1337
    c = rng.standard_normal(k).astype(np.float32)
    W = oracle.materialize_fwd(c, (rows, rowsize), (rowsize, 1), seed)
    idx = rng.integers(0, rows, size=(3, 5))
    E = oracle.embed_fwd(idx, c, rowsize, seed)
    assert E.shape == (3, 5, rowsize)
    assert np.array_equal(E, W[idx])
    # adjoint: <E(c), D> == <c, embed_bwd(D)>; repeated indices accumulate
    D = rng.standard_normal(E.shape).astype(np.float32)
    dc = oracle.embed_bwd(idx, D, k, rowsize, seed).astype(np.float64)
    lhs = float((E.astype(np.float64) * D).sum())
    assert abs(lhs - c.astype(np.float64) @ dc) < 1e-5 * abs(lhs)
    dW = np.zeros((rows, rowsize))
    np.add.at(dW, idx.reshape(-1), D.reshape(-1, rowsize).astype(np.float64))
    assert rel_l2(dc, oracle.materialize_bwd(dW.astype(np.float32), k, seed)) < 1e-5


def test_linear_layer_grad_parity_against_dense_graph(oracle):
    """The intent of the reference's check_func (benchmark.py:161-179): coef grads through the
    pseudorandom weight equal coef grads through the dense ``noise @ coef`` graph (torch autograd)."""
    torch = pytest.importorskip("torch")
    rng = np.random.default_rng(8)
    T, in_f, out_f, k, seed = 9, 12, 5, 18, 1337
    x = rng.standard_normal((T, in_f))
    dy = rng.standard_normal((T, out_f))
    for coef in (rng.standard_normal(k).astype(np.float32), rng.standard_normal((out_f, k)).astype(np.float32)):
        y = oracle.linear_fwd(x, coef, in_f, out_f, seed)
        dx, dcoef, dW = oracle.linear_bwd(x, dy, coef, in_f, out_f, seed)
        ct = torch.tensor(coef, dtype=torch.float64, requires_grad=True)
        xt = torch.tensor(x, requires_grad=True)
        if coef.ndim == 1:
            noise = torch.tensor(oracle.noise_2d_np(np.arange(out_f * in_f), np.arange(k), seed), dtype=torch.float64)
            Wt = (noise @ ct).reshape(out_f, in_f)
        else:
            N = torch.tensor(oracle.noise_2d_np(np.arange(in_f), np.arange(k), seed), dtype=torch.float64)
            Wt = ct @ N.T
        yt = xt @ Wt.T
        yt.backward(torch.tensor(dy))
        assert rel_l2(y, yt.detach().numpy()) < 1e-6
        assert rel_l2(dx, xt.grad.numpy()) < 1e-6
        assert rel_l2(dcoef, ct.grad.numpy()) < 1e-6
