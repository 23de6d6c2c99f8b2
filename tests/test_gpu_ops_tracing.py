"""The registered operators under tracing.  The reference makes its kernels ``triton_op``s so that they compose with
``torch.compile`` (src/rten_cpp/RandumbTensor.py:371, 383, 414, 1121, 1128); here every ``rten::*`` / ``rten_cpp::*`` operator
is a ``torch.library.custom_op`` with a fake (shape) implementation and, where the reference registers one, an autograd
formula.  ``torch.library.opcheck`` checks schema, fake implementation, autograd registration and AOT dispatch against real
calls; a layer compiled with the ``aot_eager`` backend (tracing, fake tensors and AOT autograd, no code generation) must give
the eager results."""
import pytest
import torch

pytestmark = pytest.mark.gpu

# dynamic shapes are left out: the projection state's size is the library's business and is asked for with concrete sizes
CHECKS = ("test_schema", "test_autograd_registration", "test_faketensor", "test_aot_dispatch_static")


@pytest.fixture(scope="module")
def ops():
    assert torch.cuda.is_available()
    from randumb_amd import ops as o

    return o


def _check(op, args, **kw):
    print("opcheck", op, flush=True)
    torch.library.opcheck(op, args, test_utils=CHECKS, **kw)


def test_opcheck_materialize_and_embedding_ops(ops):
    g = torch.Generator().manual_seed(0)
    c = torch.randn(24, generator=g).cuda()
    C = torch.randn(6, 24, generator=g).cuda()
    sb = torch.tensor([0.3]).cuda()
    _check(torch.ops.rten.materialize_fwd.default, (c.clone().requires_grad_(), [6, 10], [10, 1], 7, None, False, 0))
    _check(torch.ops.rten.materialize_fwd.default, (c.clone().requires_grad_(), [10, 6], [1, 10], 7, sb.clone().requires_grad_(), True, 0))
    _check(torch.ops.rten.materialize_fwd.default, (C.clone().requires_grad_(), [6, 10], [10, 1], 7, None, False, 10))
    dW = torch.randn(6, 10, generator=g).cuda()
    _check(torch.ops.rten.materialize_bwd.default, (dW, 24, 7, 0))
    _check(torch.ops.rten.materialize_bwd.default, (dW, 24, 7, 6))
    _check(torch.ops.rten.scale_bias_bwd.default, (dW, 7))
    idx = torch.randint(0, 50, (3, 5), generator=g).cuda()
    _check(torch.ops.rten.embed_fwd.default, (idx, c.clone().requires_grad_(), 16, 9))
    _check(torch.ops.rten.embed_bwd.default, (idx, torch.randn(3, 5, 16, generator=g).cuda(), 24, 16, 9))
    _check(torch.ops.rten_cpp.sq5_gen_2d.default, (5, 7, 3))
    _check(torch.ops.rten_cpp.materialize_fwd.default, (c, 7, 6, 10, 10, 1))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_opcheck_fused_linear_ops(ops, dtype):
    g = torch.Generator().manual_seed(1)
    T, in_f, out_f, k = 40, 64, 48, 16
    x = torch.randn(T, in_f, generator=g).to(dtype).cuda()
    dy = torch.randn(T, out_f, generator=g).to(dtype).cuda()
    C = (torch.randn(out_f, k, generator=g) * 0.1).to(dtype).cuda()
    c = (torch.randn(k, generator=g) * 0.1).to(dtype).cuda()
    bias = torch.randn(out_f, generator=g).to(dtype).cuda()
    sb = torch.tensor([0.05]).to(dtype).cuda()
    req = lambda t: t.clone().requires_grad_()
    _check(torch.ops.rten.linear_fwd.default, (req(x), req(C), in_f, out_f, in_f, 1, 5, None, req(bias)))
    _check(torch.ops.rten.linear_fwd.default, (req(x), req(c), in_f, out_f, in_f, 1, 5, req(sb), None))
    _check(torch.ops.rten.linear_bwd_dx.default, (dy, C, in_f, out_f, in_f, 1, 5, None))
    _check(torch.ops.rten.linear_bwd_dcoef.default, (dy, x, k, out_f, in_f, out_f, in_f, 1, 5, False))
    _check(torch.ops.rten.linear_bwd_dcoef.default, (dy, x, k, 0, in_f, out_f, in_f, 1, 5, True))


def test_opcheck_projected_ops(ops):
    g = torch.Generator().manual_seed(2)
    T, in_f, out_f, k = 300, 64, 48, 16
    x = torch.randn(T, in_f, generator=g).bfloat16().cuda()
    dy = torch.randn(T, out_f, generator=g).bfloat16().cuda()
    C = (torch.randn(out_f, k, generator=g) * 0.1).bfloat16().cuda()
    bias = torch.randn(out_f, generator=g).bfloat16().cuda()
    # the projection state is opaque: padding that nobody writes and the tags of the launch that wrote it are part of its bytes,
    # so two calls on the same inputs need not give the same bytes; what its consumers compute from it is checked below
    meta_only = ("test_schema", "test_autograd_registration", "test_faketensor")
    for args in ((x, k, out_f, 5, C), (x, k, out_f, 5, None)):
        print("opcheck rten.linear_project", flush=True)
        torch.library.opcheck(torch.ops.rten.linear_project.default, args, test_utils=meta_only)
    print("opcheck rten.linear_project_fwd", flush=True)
    torch.library.opcheck(torch.ops.rten.linear_project_fwd.default, (x, C, 5, bias), test_utils=meta_only)
    state = ops.linear_project(x, k, out_f, 5, C)
    _check(torch.ops.rten.linear_fwd_projected.default, (state, C, in_f, 5, bias))
    _check(torch.ops.rten.linear_bwd_dcoef_projected.default, (dy, state, k, in_f, 5), atol=1e-4, rtol=1e-4)   # fp32 atomics: order of the sums
    _check(torch.ops.rten.linear_bwd_projected.default, (dy, state, C, in_f, 5))


@pytest.mark.parametrize("dtype,matrix", [(torch.bfloat16, True), (torch.float32, True), (torch.float32, False)])
def test_compiled_layer_matches_eager(ops, dtype, matrix):
    """SillyLinear forward + backward traced by torch.compile (aot_eager: Dynamo, fake tensors, AOT autograd; graph breaks
    allowed) against the same layer run eagerly: bf16 matrix-coef takes the projected operators, fp32 the rten::linear_fwd
    family, vector-coef the tensor subclass's dispatch."""
    import randumb_amd as ra

    print(f"case compiled layer {dtype} matrix={matrix}", flush=True)
    torch._dynamo.reset()
    in_f, out_f, k, T = 128, 256, 32, 300
    layer = ra.SillyLinear(in_f, out_f, [k, k], [11, 12], bias=False, matrix_coef=matrix).to(dtype).cuda()
    with torch.no_grad():
        g = torch.Generator().manual_seed(3)
        layer.weight_coef.copy_((torch.randn(layer.weight_coef.shape, generator=g) * 0.05).to(dtype))
        layer.weight_scale_bias.zero_()
    x0 = torch.randn(T, in_f, generator=torch.Generator().manual_seed(4)).to(dtype).cuda()

    def run(fn):
        layer.zero_grad(set_to_none=True)
        x = x0.clone().requires_grad_()
        y = fn(x)
        (y.float() ** 2).sum().backward()
        torch.cuda.synchronize()
        return y.detach(), x.grad.detach(), layer.weight_coef.grad.detach()

    eager = run(layer)
    traced = []

    def backend(gm, example_inputs):   # aot_eager, after a look at what Dynamo captured (autograd functions are sub-graphs)
        from torch._dynamo.backends.debugging import aot_eager

        for mod in gm.modules():
            if isinstance(mod, torch.fx.GraphModule):
                traced.extend(str(n.target) for n in mod.graph.nodes if n.op == "call_function")
        return aot_eager(gm, example_inputs)

    compiled_layer = torch.compile(layer, backend=backend, fullgraph=False)
    for _ in range(2):   # the second call runs the cached graph
        got = run(compiled_layer)
        for name, a, b in zip(("y", "dx", "dcoef"), got, eager):
            assert a.shape == b.shape and a.dtype == b.dtype, name
            # the projected form's dcoef is bit-reproducible, as are y and dx everywhere; vector-coef sums may differ in order
            tol = 0.0 if matrix else 1e-5
            err = float((a.float() - b.float()).norm() / b.float().norm().clamp_min(1e-30))
            assert err <= tol, f"{name}: compiled differs from eager by {err}"
    # the registered operators are what was traced (not an eager fall-back behind a graph break).  The vector-coef layer
    # reaches its operator inside the tensor subclass's __torch_dispatch__, at run time, below what Dynamo records.
    if matrix:
        want = "rten.linear_project_fwd" if dtype == torch.bfloat16 else "rten.linear_fwd"
        assert any(want in t for t in traced), (want, sorted(set(traced)))
