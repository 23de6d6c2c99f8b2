"""GPU behaviour of the tensor subclass, the autograd bridge and the layers against the CPU oracle / a dense
fp64 autograd graph.  Tolerances: fp32 1e-5, bf16 2e-2 (relative L2)."""
import math

import numpy as np
import pytest
import torch
import torch.nn.functional as F

pytestmark = pytest.mark.gpu
F32_TOL, BF16_TOL = 1e-5, 2e-2


def rel_l2(a, b):
    a = np.asarray(a, dtype=np.float64)
    b = np.asarray(b, dtype=np.float64)
    return float(np.linalg.norm(a - b) / max(np.linalg.norm(b), 1e-30))


def cpu(t):
    return t.detach().float().cpu().numpy()


@pytest.fixture(scope="module")
def ra():
    assert torch.cuda.is_available()
    import randumb_amd

    return randumb_amd


def test_check_func_parity(ra, oracle):
    """What the reference's check_func sets out to verify (benchmark.py:132-179), with assertions."""
    print("case check_func", flush=True)
    n, m, seed = 18, 18, 1337
    g = torch.Generator().manual_seed(0)
    coefs = torch.randn(m, generator=g)
    noise = torch.tensor(oracle.noise_2d(n, m, seed), dtype=torch.float64)
    true_coefs = coefs.double().requires_grad_()
    true_out = (noise @ true_coefs).reshape(3, 6)
    rt_coef = coefs.cuda().requires_grad_()
    rt = ra.CreateRandumbTensor(rt_coef, seed, (3, 6))
    assert rel_l2(cpu(rt.get_materialized()), true_out.detach().numpy()) < F32_TOL
    assert np.array_equal(cpu(rt.get_noise_matrix()).view(np.uint32), oracle.noise_2d(n, m, seed).view(np.uint32))
    x = torch.randn(6, 12, generator=g)
    lin = torch.nn.Linear(12, 8)
    true_eqn = F.linear(true_out @ x.double(), lin.weight.double(), lin.bias.double()).sum()
    true_eqn.backward()
    lin_gpu = torch.nn.Linear(12, 8).cuda()
    lin_gpu.load_state_dict(lin.state_dict())
    rt_eqn = lin_gpu(rt @ x.cuda()).sum()
    rt_eqn.backward()
    assert abs(float(rt_eqn) - float(true_eqn)) < 1e-4 * max(1.0, abs(float(true_eqn)))
    assert rel_l2(cpu(rt_coef.grad), true_coefs.grad.numpy()) < F32_TOL
    assert rt._tensor is None  # freed after every op


def test_dispatch_semantics(ra, oracle):
    print("case dispatch", flush=True)
    seed = 47
    c = torch.randn(16).cuda()
    rt = ra.CreateRandumbTensor(c, seed, (6, 10))
    W = oracle.materialize_fwd(cpu(c), (6, 10), (10, 1), seed)
    assert rel_l2(cpu(rt + 0), W) < F32_TOL                     # generic op: materialise, run, free
    assert rel_l2(cpu(rt.t() + 0), W.T) < F32_TOL               # lazy transpose follows the original linear index
    assert rel_l2(cpu(rt.view(10, 6) + 0), W.reshape(10, 6)) < F32_TOL
    assert rel_l2(cpu(rt.view(2, 3, 10).permute(2, 0, 1) + 0), W.reshape(2, 3, 10).transpose(2, 0, 1)) < F32_TOL
    assert (rt.to(torch.bfloat16) + 0).dtype == torch.bfloat16
    x = torch.randn(5, 10).cuda()
    want = cpu(x).astype(np.float64) @ W.T.astype(np.float64)
    z = torch.randn(10, 4).cuda()
    # a vector-coef tensor: materialise-then-matmul (the reference's data flow) unless the fused kernels are asked for
    assert not ra.RandumbTensor.FUSED_MM_VECTOR
    assert rel_l2(cpu(x @ rt.t()), want) < F32_TOL
    ra.RandumbTensor.FUSED_MM_VECTOR = True
    try:
        assert rt._fused_ok(x)
        assert rel_l2(cpu(x @ rt.t()), want) < F32_TOL              # fused mat1 @ tensor
        assert rel_l2(cpu(F.linear(x, rt)), want) < F32_TOL
        assert rel_l2(cpu(rt @ z), W.astype(np.float64) @ cpu(z).astype(np.float64)) < F32_TOL   # tensor @ mat2
        ra.RandumbTensor.FUSED_MM = False
        try:
            assert not rt._fused_ok(x)
            assert rel_l2(cpu(x @ rt.t()), want) < F32_TOL
        finally:
            ra.RandumbTensor.FUSED_MM = True
    finally:
        ra.RandumbTensor.FUSED_MM_VECTOR = False
    assert not rt._fused_ok(x)
    # fused random bias
    sb = torch.tensor([0.3]).cuda()
    rtb = ra.CreateRandumbTensor(c, seed, (6, 10), sb, True)
    Wb = oracle.materialize_fwd(cpu(c), (6, 10), (10, 1), seed, scale_bias=0.3)
    assert rel_l2(cpu(rtb + 0), Wb) < F32_TOL
    assert rel_l2(cpu(x @ rtb.t()), cpu(x).astype(np.float64) @ Wb.T.astype(np.float64)) < F32_TOL


def test_matrix_coef_tensor_dispatch(ra, oracle):
    print("case matrix-coef dispatch", flush=True)
    seed, out_f, in_f, k = 5, 40, 24, 16
    C = torch.randn(out_f, k).cuda().requires_grad_()
    rt = ra.CreateRandumbTensor(C, seed, (out_f, in_f))
    W = oracle.materialize_fwd(cpu(C), (out_f, in_f), (in_f, 1), seed, row_len=in_f).astype(np.float64)
    x = torch.randn(9, in_f).cuda().requires_grad_()
    y = F.linear(x, rt)
    assert rel_l2(cpu(y), cpu(x).astype(np.float64) @ W.T) < F32_TOL
    dy = torch.randn(9, out_f).cuda()
    y.backward(dy)
    dx, dC, _ = oracle.linear_bwd(cpu(x), cpu(dy), cpu(C), in_f, out_f, seed)
    assert rel_l2(cpu(x.grad), dx) < F32_TOL and rel_l2(cpu(C.grad), dC) < F32_TOL and C.grad.shape == C.shape


def _dense_mlp_reference(oracle, x, coefs, seeds, dims, matrix, target, lr):
    """fp64 autograd graph through the dense noise matrices: loss, coefficient grads, coefficients after one SGD step."""
    ps = [torch.tensor(c, dtype=torch.float64, requires_grad=True) for c in coefs]
    h = torch.tensor(x, dtype=torch.float64)
    for li, ((in_f, out_f), c, seed) in enumerate(zip(dims, ps, seeds)):
        k = c.shape[-1]
        if matrix:
            N = torch.tensor(oracle.noise_2d(in_f, k, seed), dtype=torch.float64)
            W = c @ N.T
        else:
            N = torch.tensor(oracle.noise_2d(out_f * in_f, k, seed), dtype=torch.float64)
            W = (N @ c).reshape(out_f, in_f)
        h = h @ W.T
        if li == 0:
            h = torch.relu(h)
    loss = ((h - torch.tensor(target, dtype=torch.float64)) ** 2).mean()
    loss.backward()
    return h.detach().numpy(), float(loss), [p.grad.numpy() for p in ps], [(p - lr * p.grad).detach().numpy() for p in ps]


@pytest.mark.parametrize("matrix,fused", [(False, False), (True, True), (False, True), (True, False)])
def test_mnist_shaped_mlp_forward_backward_sgd(ra, oracle, matrix, fused):
    """784 -> 256 -> 10, k = 64, seeds 1337 / 1338, batch 128 of x ~ U[0, 1], fp32: forward, backward, one SGD step."""
    print(f"case mlp matrix={matrix} fused={fused}", flush=True)
    g = torch.Generator().manual_seed(0)
    dims, seeds, k, lr = [(784, 256), (256, 10)], [1337, 1338], 64, 0.1
    x = torch.rand(128, 784, generator=g)
    target = torch.randn(128, 10, generator=g)
    layers, coefs = [], []
    for (in_f, out_f), seed in zip(dims, seeds):
        l = ra.SillyLinear(in_f, out_f, [k, k], [seed, seed + 100], bias=False, matrix_coef=matrix, fused=fused)
        std = math.sqrt(1.0 / 3.0) / math.sqrt(in_f)  # kaiming_uniform(a=sqrt(5)) standard deviation
        with torch.no_grad():
            l.weight_coef.copy_(torch.randn(l.weight_coef.shape, generator=g) * math.sqrt(3 * std**2 / k))
            l.weight_scale_bias.zero_()
        coefs.append(l.weight_coef.detach().numpy().copy())
        layers.append(l.cuda())
    model = torch.nn.Sequential(layers[0], torch.nn.ReLU(), layers[1])
    opt = torch.optim.SGD(model.parameters(), lr=lr)
    out = model(x.cuda())
    loss = ((out - target.cuda()) ** 2).mean()
    loss.backward()
    want_out, want_loss, want_grads, want_new = _dense_mlp_reference(oracle, x.numpy(), coefs, seeds, dims, matrix, target.numpy(), lr)
    assert rel_l2(cpu(out), want_out) < F32_TOL
    assert abs(float(loss) - want_loss) < 1e-5 * want_loss
    for l, wg in zip(layers, want_grads):
        assert l.weight_coef.grad.shape == l.weight_coef.shape and rel_l2(cpu(l.weight_coef.grad), wg) < F32_TOL
    opt.step()
    for l, wn in zip(layers, want_new):
        assert rel_l2(cpu(l.weight_coef), wn) < F32_TOL


def test_default_layer_with_biases_trains(ra, oracle):
    """Reference default: zero coefficients + fused random bias on weight and bias tensors; every parameter gets a gradient."""
    print("case default layer", flush=True)
    for matrix in (False, True):
        l = ra.SillyLinear(32, 12, [8, 8], [3, 4], bias=True, rt_bias=True, matrix_coef=matrix).cuda()
        x = torch.randn(5, 32).cuda()
        y = l(x)
        sW, sB = float(l.weight_scale_bias), float(l.bias_scale_bias)
        W = sW * oracle.noise_1d(12 * 32, 3).reshape(12, 32).astype(np.float64)
        b = sB * oracle.noise_1d(12, 4).astype(np.float64)
        assert rel_l2(cpu(y), cpu(x).astype(np.float64) @ W.T + b) < F32_TOL
        y.sum().backward()
        for name, p in l.named_parameters():
            assert p.grad is not None and p.grad.shape == p.shape, name
        dW = np.ones((5, 12)).T @ cpu(x).astype(np.float64)
        want_ds = float((dW.reshape(-1) * oracle.noise_1d(12 * 32, 3)).sum())
        assert abs(float(l.weight_scale_bias.grad) - want_ds) < 1e-4 * max(1.0, abs(want_ds))


def test_bf16_layer_matches_oracle(ra, oracle):
    print("case bf16 layer", flush=True)
    g = torch.Generator().manual_seed(3)
    in_f, out_f, k, seed, T = 768, 512, 256, 0, 512   # k*(in+out) < in*out: the factored products are the cheaper form
    l = ra.SillyLinear(in_f, out_f, [k, k], [seed, 1], bias=False, matrix_coef=True)
    with torch.no_grad():
        l.weight_coef.copy_(torch.randn(out_f, k, generator=g) * math.sqrt(3 * 0.02**2 / k))
        l.weight_scale_bias.zero_()
    l = l.to(torch.bfloat16).cuda()
    x = torch.randn(4, T // 4, in_f, generator=g).bfloat16().cuda().requires_grad_()
    dy = torch.randn(4, T // 4, out_f, generator=g).bfloat16().cuda()
    y = l(x)
    assert y.shape == (4, T // 4, out_f) and y.dtype == torch.bfloat16
    # a matrix-coef bf16 layer without the fused random bias takes the projected form: z = x.N^T saved for the backward pass
    assert "ProjectedLinear" in str(y.grad_fn.next_functions[0][0])
    y.backward(dy)
    xn, dyn, Cn = cpu(x).reshape(T, in_f), cpu(dy).reshape(T, out_f), cpu(l.weight_coef)
    assert rel_l2(cpu(y).reshape(T, out_f), oracle.linear_fwd(xn, Cn, in_f, out_f, seed)) < BF16_TOL
    dx, dC, _ = oracle.linear_bwd(xn, dyn, Cn, in_f, out_f, seed)
    assert rel_l2(cpu(x.grad).reshape(T, in_f), dx) < BF16_TOL
    assert l.weight_coef.grad.dtype == torch.bfloat16 and rel_l2(cpu(l.weight_coef.grad), dC) < BF16_TOL


def test_bf16_layer_with_fused_random_bias_takes_the_projected_form(ra, oracle):
    """The reference's default layer (fused random bias s.R on the weight, SillyLayers.py:122-133) in bf16 with non-zero
    coefficients: the low-rank share through the projected entry points (z saved by the forward pass), the random-bias share
    through kernels of its own in both directions, the gradient of s from the input gradient's pass; all against the oracle."""
    print("case bf16 layer with scale_bias", flush=True)
    g = torch.Generator().manual_seed(8)
    in_f, out_f, k, seed, T = 512, 384, 128, 5, 640
    l = ra.SillyLinear(in_f, out_f, [k, k], [seed, 1], bias=False, rt_bias=True, matrix_coef=True)
    with torch.no_grad():
        l.weight_coef.copy_(torch.randn(out_f, k, generator=g) * 0.02)
        l.weight_scale_bias.fill_(0.0625)
    l = l.to(torch.bfloat16).cuda()
    x = torch.randn(T, in_f, generator=g).bfloat16().cuda().requires_grad_()
    dy = torch.randn(T, out_f, generator=g).bfloat16().cuda()
    y = l(x)
    assert "ProjectedLinear" in str(y.grad_fn) or "ProjectedLinear" in str(y.grad_fn.next_functions[0][0])
    y.backward(dy)
    xn, dyn, Cn = cpu(x), cpu(dy), cpu(l.weight_coef)
    assert rel_l2(cpu(y), oracle.linear_fwd(xn, Cn, in_f, out_f, seed, scale_bias=0.0625)) < BF16_TOL
    dx, dC, dW = oracle.linear_bwd(xn, dyn, Cn, in_f, out_f, seed, scale_bias=0.0625)
    assert rel_l2(cpu(x.grad), dx) < BF16_TOL
    assert rel_l2(cpu(l.weight_coef.grad), dC) < BF16_TOL
    want_ds = float(oracle.scale_bias_bwd(dW.astype(np.float32), seed)[0])
    assert abs(float(l.weight_scale_bias.grad) - want_ds) < BF16_TOL * max(abs(want_ds), float(np.linalg.norm(dW)))
    # only the scale wants a gradient: still computed (from the random-bias share of an input gradient nobody asked for)
    l.zero_grad(set_to_none=True)
    l.weight_coef.requires_grad_(False)
    l(x.detach()).backward(dy)
    assert abs(float(l.weight_scale_bias.grad) - want_ds) < BF16_TOL * max(abs(want_ds), float(np.linalg.norm(dW)))


def test_conv2d_layers_match_a_dense_autograd_graph(ra, oracle):
    """Two convolution layers with pseudorandom kernels (the front of the reference's MNIST net, mnist.py:55-84) against the
    same convolutions on dense kernels built from the oracle, in fp64 on the CPU: output, input gradient, and the gradient
    of every coefficient vector and scale."""
    print("case conv2d", flush=True)
    g = torch.Generator().manual_seed(5)
    ints, seeds = ra.stepgen(48, 0), ra.stepgen(77, 1)
    c1 = ra.SillyConv2d(1, 8, int_dim=ints, seed=seeds, kernel_size=3, stride=1, rt_bias=True)
    c2 = ra.SillyConv2d(8, 16, int_dim=ints, seed=seeds, kernel_size=3, stride=2, padding=1, rt_bias=True)
    with torch.no_grad():
        for c in (c1, c2):
            c.weight_coef.copy_(torch.randn(48, generator=g) * 0.1)
            c.bias_coef.copy_(torch.randn(48, generator=g) * 0.1)
    c1, c2 = c1.cuda(), c2.cuda()
    x = torch.rand(4, 1, 12, 12, generator=g)
    xg = x.cuda().requires_grad_()
    y = c2(F.relu(c1(xg)))
    assert y.shape == (4, 16, 5, 5) and c1.weight._tensor is None
    y.square().sum().backward()

    # dense twin: W_flat = Noise(seed) @ coef + scale * noise1d(seed), element index = offset in the contiguous kernel
    leaves, kernels = {}, {}
    for name, c, seed_w, seed_b in (("c1", c1, 77, 78), ("c2", c2, 79, 80)):
        for kind, rt, seed in (("weight", c.weight, seed_w), ("bias", c.bias, seed_b)):
            n = rt.numel()
            coef = torch.tensor(cpu(getattr(c, kind + "_coef")), dtype=torch.float64, requires_grad=True)
            sb = torch.tensor(cpu(getattr(c, kind + "_scale_bias")), dtype=torch.float64, requires_grad=True)
            noise = torch.tensor(oracle.noise_2d(n, 48, seed), dtype=torch.float64)
            bias = torch.tensor(oracle.noise_1d(n, seed), dtype=torch.float64)
            kernels[name, kind] = (noise @ coef + sb * bias).reshape(tuple(rt.shape))
            leaves[name, kind] = (coef, sb)
    xd = x.double().requires_grad_()
    yd = F.conv2d(F.relu(F.conv2d(xd, kernels["c1", "weight"], kernels["c1", "bias"])), kernels["c2", "weight"], kernels["c2", "bias"],
                  stride=2, padding=1)
    yd.square().sum().backward()
    assert rel_l2(cpu(y), yd.detach().numpy()) < 1e-5
    assert rel_l2(cpu(xg.grad), xd.grad.numpy()) < 1e-4
    for (name, kind), (coef, sb) in leaves.items():
        c = c1 if name == "c1" else c2
        assert rel_l2(cpu(getattr(c, kind + "_coef").grad), coef.grad.numpy()) < 1e-4, (name, kind)
        assert rel_l2(cpu(getattr(c, kind + "_scale_bias").grad), sb.grad.numpy()) < 1e-4, (name, kind)


def test_mnist_conv_net_trains(ra):
    """The reference's MNIST net (mnist/mnist.py:55-84: two pseudorandom convolutions, two pseudorandom linears) on a fixed
    synthetic batch: every parameter gets a finite gradient and a few SGD steps lower the loss."""
    print("case conv net", flush=True)
    torch.manual_seed(0)
    ints, seeds = ra.stepgen(64, 0), ra.stepgen(1337, 1)

    class Net(torch.nn.Module):
        def __init__(self):
            super().__init__()
            self.conv1 = ra.SillyConv2d(1, 32, int_dim=ints, seed=seeds, kernel_size=3, stride=1, rt_bias=True)
            self.conv2 = ra.SillyConv2d(32, 64, int_dim=ints, seed=seeds, kernel_size=3, stride=1, rt_bias=True)
            self.fc1 = ra.SillyLinear(9216, 128, ints, seeds, bias=False, rt_bias=True)
            self.fc2 = ra.SillyLinear(128, 10, ints, seeds, bias=False, rt_bias=True)

        def forward(self, x):
            x = F.max_pool2d(F.relu(self.conv2(F.relu(self.conv1(x)))), 2)
            return F.log_softmax(self.fc2(F.relu(self.fc1(torch.flatten(x, 1)))), dim=1)

    net = Net().cuda()
    assert [l.seed for l in (net.conv1, net.conv2, net.fc1, net.fc2)] == [[1337, 1338], [1339, 1340], [1341, 1342], [1343, 1344]]
    x, target = torch.rand(16, 1, 28, 28).cuda(), torch.randint(0, 10, (16,)).cuda()
    # a coefficient moves every weight that shares it, so its gradient is large: steps of fixed length along the gradient
    params, losses = list(net.parameters()), []
    for _ in range(6):
        net.zero_grad()
        loss = F.nll_loss(net(x), target)
        loss.backward()
        for name, p in net.named_parameters():
            assert p.grad is not None and torch.isfinite(p.grad).all(), name
        norm = torch.sqrt(sum((p.grad.double() ** 2).sum() for p in params)).item()
        with torch.no_grad():
            for p in params:
                p -= (0.02 / norm) * p.grad
        losses.append(float(loss.detach()))
    assert losses[-1] < losses[0], losses


def test_embedding_layer(ra, oracle):
    print("case embedding", flush=True)
    e = ra.SillyEmbedding(1000, 48, [32], [9], device="cuda")
    idx = torch.randint(0, 1000, (4, 7)).cuda()
    out = e(idx)
    want = oracle.embed_fwd(cpu(idx).astype(np.int64), cpu(e.weight_coef), 48, 9)
    assert out.shape == (4, 7, 48) and rel_l2(cpu(out), want) < F32_TOL
    D = torch.randn(4, 7, 48).cuda()
    out.backward(D)
    assert rel_l2(cpu(e.weight_coef.grad), oracle.embed_bwd(cpu(idx).astype(np.int64), cpu(D), 32, 48, 9)) < F32_TOL


def test_rt_mm_and_cpp_ops(ra, oracle):
    print("case rt_mm", flush=True)
    L, P, Q, k, seed = 33, 20, 28, 12, 1337
    c = torch.randn(k).cuda()
    mat1 = torch.randn(L, P).cuda()
    W = oracle.materialize_fwd(cpu(c), (P, Q), (Q, 1), seed).astype(np.float64)
    got = ra.rt_mm(mat1, c, (P, Q), (Q, 1), seed, None, False)
    assert got.shape == (L, Q) and rel_l2(cpu(got), cpu(mat1).astype(np.float64) @ W) < F32_TOL
    got2 = torch.ops.rten_cpp.materialize_fwd(c, seed, P, Q, Q, 1)
    assert rel_l2(cpu(got2), W) < F32_TOL
    n = torch.ops.rten_cpp.sq5_gen_2d(7, 5, seed)
    assert np.array_equal(cpu(n).view(np.uint32), oracle.noise_2d(7, 5, seed).view(np.uint32))
    w = torch.ops.rten.materialize_fwd(c.requires_grad_(), [P, Q], [Q, 1], seed, None, False)
    w.sum().backward()
    assert rel_l2(cpu(c.grad), oracle.materialize_bwd(np.ones(P * Q, np.float32), k, seed)) < F32_TOL


def test_step_is_graph_capturable(ra):
    """The forward and backward calls of a layer record into a HIP graph (no allocation, no memset node: the library clears
    with a fill kernel) and every replay, with eager work in between, gives the eager result."""
    print("case graph capture", flush=True)
    from randumb_amd import hip

    T, in_f, out_f, k, seed = 512, 256, 384, 64, 5
    g = torch.Generator().manual_seed(1)
    x = torch.randn(T, in_f, generator=g).bfloat16().cuda()
    dy = torch.randn(T, out_f, generator=g).bfloat16().cuda()
    C = (torch.randn(out_f, k, generator=g) * 0.05).bfloat16().cuda()

    def step():
        z = hip.linear_project(x, k, out_f, seed)
        y = hip.linear_fwd_projected(z, C, in_f, seed)
        dx, dc = hip.linear_bwd_projected(dy, z, C, in_f, seed)
        return y, dx, dc

    want = [t.clone() for t in step()]
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        got = step()
    for i in range(4):
        for t in got:
            t.fill_(3.0)
        _ = step()                      # eager work between replays
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(got[0], want[0]) and torch.equal(got[1], want[1]), f"replay {i}"
        assert float((got[2] - want[2]).abs().max()) <= 1e-5 * float(want[2].abs().max()), f"replay {i}"


def test_one_launch_forms_replay_in_a_graph_on_new_inputs(ra):
    """The launches whose later blocks wait for tags of their earlier blocks (projection + forward product in bf16, contraction +
    expansion in fp32 with small k) carry the tag they were recorded with: replayed from a HIP graph on inputs that changed in
    between, every replay must wait again and give that input's result (the consumers clear the tags they have seen)."""
    print("case graph replay of the one-launch forms", flush=True)
    from randumb_amd import hip

    g = torch.Generator().manual_seed(2)
    T, in_f, out_f, k, seed = 1024, 256, 512, 64, 3
    xs = [torch.randn(T, in_f, generator=g).bfloat16().cuda() for _ in range(4)]
    C = (torch.randn(out_f, k, generator=g) * 0.05).bfloat16().cuda()
    want = [hip.linear_project_fwd(x, C, seed)[0].clone() for x in xs]
    x = xs[0].clone()
    T3, in3, out3, k3 = 16, 4096, 4096, 16
    x3s = [torch.randn(T3, in3, generator=g).cuda() for _ in range(4)]
    C3 = (torch.randn(out3, k3, generator=g) * 0.05).cuda()
    want3 = [hip.linear_fwd(v, C3, in3, out3, in3, 1, seed).clone() for v in x3s]
    x3 = x3s[0].clone()
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        y, _state = hip.linear_project_fwd(x, C, seed)
        y3 = hip.linear_fwd(x3, C3, in3, out3, in3, 1, seed)
    for i in (1, 2, 3, 0, 2):
        x.copy_(xs[i])
        x3.copy_(x3s[i])
        y.fill_(7.0)
        y3.fill_(7.0)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(y, want[i]), f"bf16 forward, input {i}"
        assert torch.equal(y3, want3[i]), f"fp32 small-k forward, input {i}"
