"""Compiled (torch.compile, fullgraph=True) versus eager, on the GPU: same kernels behind registered ops, so results are
bit-identical. Backend "aot_eager": the graph is captured and partitioned by AOT autograd, nothing is re-generated
(the reference's tests compile every op with fullgraph=True, e.g. scattermoe_test.py:80-81, rmsnorm_test.py:34)."""

import pytest
import torch

import cute_kernels as ck

pytestmark = pytest.mark.gpu


@pytest.fixture(autouse=True)
def _fresh_dynamo():
    """Every case compiles a new module instance of the same code objects: start from an empty cache so that dynamo's
    per-function recompile limit is not what a later case trips over."""
    torch._dynamo.reset()
    yield


def _compile(fn):
    return torch.compile(fn, fullgraph=True, backend="aot_eager")


def test_count_compiled(device):
    ids = torch.randint(0, 64, (65536,), dtype=torch.int32, device=device)
    out = _compile(lambda i: ck.continuous_count_cute(i, 64))(ids)
    assert out.dtype == torch.uint32 and torch.equal(out.cpu().long(), torch.bincount(ids.cpu().long(), minlength=64))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_swiglu_and_norms_compiled(device, dtype):
    g = torch.Generator().manual_seed(0)
    x = torch.randn(300, 512, generator=g).to(dtype).to(device)
    y = torch.randn(300, 512, generator=g).to(dtype).to(device)
    w = torch.randn(512, generator=g).to(dtype).to(device)
    cases = {
        "swiglu": (lambda a, b, c: ck.swiglu_cute(a, b), 2),
        "swiglu_packed": (lambda a, b, c: ck.swiglu_packed_cute(a), 1),
        "rmsnorm": (lambda a, b, c: ck.rmsnorm_cute(a, c, 1e-5), 3),
        "rmsnorm_me": (lambda a, b, c: ck.rmsnorm_cute(a, None, None, memory_efficient=True), 1),
        "softmax": (lambda a, b, c: ck.softmax_cute(a, 0.7), 1),
        "frn": (lambda a, b, c: sum(t.float() for t in ck.fused_residual_add_rmsnorm_cute(a, b, c, 1e-5, 0.9)), 3),
        "frn_me": (lambda a, b, c: ck.fused_residual_add_rmsnorm_cute(a, b, None, 1e-5, None, True)[0], 2),
    }
    for name, (fn, _) in cases.items():
        eager_in = [t.clone().requires_grad_() for t in (x, y, w)]
        comp_in = [t.clone().requires_grad_() for t in (x, y, w)]
        z = fn(*eager_in)
        zc = _compile(fn)(*comp_in)
        assert torch.equal(z, zc), name
        z.float().square().sum().backward()
        zc.float().square().sum().backward()
        for a, b in zip(eager_in, comp_in):
            assert (a.grad is None) == (b.grad is None), name
            if a.grad is not None:
                assert torch.equal(a.grad, b.grad), name


@pytest.mark.parametrize("add_bias", [False, True])
@pytest.mark.parametrize("act,is_glu", [(ck.swiglu_packed_cute, True), (torch.nn.GLU(), True), (torch.nn.GELU("tanh"), False)])
def test_moe_layer_compiled(device, act, is_glu, add_bias):
    torch.manual_seed(1)
    moe = ck.MoE(8, 2, 128, 256, act, is_glu, add_bias, 0.02).to(torch.bfloat16).to(device)
    if add_bias:
        with torch.no_grad():
            moe.c_fc.bias.normal_(0, 0.1)
            moe.c_proj.bias.normal_(0, 0.1)
    x = torch.randn(512, 128, dtype=torch.bfloat16, device=device)
    xe, xc = x.clone().requires_grad_(), x.clone().requires_grad_()
    y, logits = moe(xe)
    y.float().square().sum().backward()
    eager_grads = {n: p.grad.clone() for n, p in moe.named_parameters()}
    for p in moe.parameters():
        p.grad = None
    compiled = _compile(moe)
    yc, logits_c = compiled(xc)
    yc.float().square().sum().backward()
    assert torch.equal(y, yc) and torch.equal(logits, logits_c)
    # Everything that does not pass through d_gates is bit-identical. The eager layer hands d_gates from the expert
    # block to the router in fp32 (a side channel next to autograd); a traced graph carries it in the gates' dtype, as
    # the reference does (ops.py:214). So the router's share of x.grad and gate.weight.grad differ by that one rounding.
    for n, p in moe.named_parameters():
        if n == "gate.weight":
            torch.testing.assert_close(eager_grads[n].float(), p.grad.float(), rtol=2e-2, atol=2e-2 * float(p.grad.float().abs().max()))
        else:
            assert torch.equal(eager_grads[n], p.grad), n
    torch.testing.assert_close(xe.grad.float(), xc.grad.float(), rtol=2e-2, atol=2e-2 * float(xc.grad.float().abs().max()))
    # inference: nothing is saved, nothing breaks
    with torch.no_grad():
        assert torch.equal(compiled(x)[0], moe(x)[0])


@pytest.mark.timeout(900)
@pytest.mark.parametrize("act,is_glu", [(ck.swiglu_packed_cute, True), (torch.nn.GELU("tanh"), False)])
def test_moe_layer_compiled_with_the_default_backend(device, act, is_glu):
    """torch.compile(moe, fullgraph=True) with no backend argument (inductor), as the reference's own layer test compiles
    it (scattermoe_test.py:80-81). The registered operators stay opaque calls into the library; what inductor
    re-generates around them (the router's matmul and casts, the activation callable of the unfused path) may round
    differently from eager by one step of the 16-bit type, hence rtol = atol = 2e-2 relative to each tensor's largest
    element instead of bit equality."""
    torch.manual_seed(1)
    moe = ck.MoE(8, 2, 128, 256, act, is_glu, False, 0.02).to(torch.bfloat16).to(device)
    x = torch.randn(512, 128, dtype=torch.bfloat16, device=device)
    xe, xc = x.clone().requires_grad_(), x.clone().requires_grad_()
    y, logits = moe(xe)
    y.float().square().sum().backward()
    eager_grads = {n: p.grad.clone() for n, p in moe.named_parameters()}
    for p in moe.parameters():
        p.grad = None
    compiled = torch.compile(moe, fullgraph=True)
    yc, logits_c = compiled(xc)
    yc.float().square().sum().backward()

    def close(a, b, what):
        torch.testing.assert_close(a.float(), b.float(), rtol=2e-2, atol=2e-2 * float(b.float().abs().max()), msg=lambda m: what + ": " + m)

    close(logits_c, logits, "logits")
    close(yc, y, "output")
    close(xc.grad, xe.grad, "x.grad")
    for n, p in moe.named_parameters():
        close(p.grad, eager_grads[n], n)


class _NormGluNorm(torch.nn.Module):  # examples/cute_inductor.py:21-33 of the reference, with a packed SwiGLU in the middle
    def __init__(self) -> None:
        super().__init__()
        self.norm1 = torch.nn.RMSNorm(256, eps=1e-5)
        self.linear = torch.nn.Linear(256, 1024)
        self.norm2 = torch.nn.RMSNorm(512, eps=1e-6)  # explicit: torch's GPU kernel evaluates a None eps in fp32, rmsnorm_cute in x.dtype

    def forward(self, x):
        x = self.linear(self.norm1(x))
        up, gate = x.chunk(2, dim=-1)
        return self.norm2(up * torch.nn.functional.silu(gate))


@pytest.mark.parametrize("then_inductor", [False, True])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_cute_inductor_rewrites_match_the_torch_model(device, dtype, then_inductor):
    """The model compiled through CuteInductor (rmsnorm_cute + swiglu_packed_cute swapped in) against the same model run
    by torch eagerly: outputs and every gradient within the elementwise-kernel tolerances (fp32 1e-5; bf16 one rounding
    step of values of order 1: atol 2e-2, rtol 2e-2)."""
    from cute_kernels import CuteInductor

    torch.manual_seed(0)
    model = _NormGluNorm().to(dtype).to(device)
    x = torch.randn(333, 256, device=device, dtype=dtype)
    g = torch.randn(333, 512, device=device, dtype=dtype)
    x_ref = x.clone().requires_grad_()
    model(x_ref).backward(g)
    want = [x_ref.grad] + [p.grad.clone() for p in model.parameters()]
    want_y = model(x)
    for p in model.parameters():
        p.grad = None

    seen = []
    inductor = CuteInductor(use_torch_inductor_after_cute_inductor=then_inductor)

    def backend(gm, example_inputs):
        run = inductor.compiler(gm, example_inputs)
        seen.extend(n.target for n in gm.graph.nodes if n.op == "call_function")
        return run

    compiled = torch.compile(model, backend=backend, fullgraph=True)
    x_got = x.clone().requires_grad_()
    y = compiled(x_got)
    assert seen.count(ck.rmsnorm_cute) == 2 and seen.count(ck.swiglu_packed_cute) == 1
    y.backward(g)
    got = [x_got.grad] + [p.grad for p in model.parameters()]
    tol = dict(atol=1e-5, rtol=1e-5) if dtype == torch.float32 else dict(atol=2e-2, rtol=2e-2)
    torch.testing.assert_close(y, want_y, **tol)
    for a, b in zip(got, want):
        # weight gradients sum 333 rows: compare in units of the gradient's own scale
        scale = max(1.0, float(b.float().abs().max()))
        torch.testing.assert_close(a.float() / scale, b.float() / scale, **tol)


def test_layer_on_the_reference_interface_compiled(device):
    """A layer whose _compute_experts calls the expert linears the way the reference's accelerated layer does
    (scattered_experts on sort / bincount / cumsum results) under torch.compile(fullgraph=True, backend="aot_eager"):
    same kernels as eager, so everything that does not pass through d_gates is bit-identical (see the layer test above)."""
    from test_compile_trace import _LayerOnTheReferenceInterface

    torch.manual_seed(3)
    moe = _LayerOnTheReferenceInterface(8, 2, 128, 256, ck.swiglu_packed_cute, True, False, 0.02).to(torch.bfloat16).to(device)
    x = torch.randn(700, 128, dtype=torch.bfloat16, device=device)
    xe, xc = x.clone().requires_grad_(), x.clone().requires_grad_()
    y, _ = moe(xe)
    y.float().square().sum().backward()
    eager_grads = {n: p.grad.clone() for n, p in moe.named_parameters()}
    for p in moe.parameters():
        p.grad = None
    compiled = torch.compile(moe, fullgraph=True, backend="aot_eager")
    yc, _ = compiled(xc)
    assert torch.equal(yc, y)
    yc.float().square().sum().backward()
    for n, p in moe.named_parameters():
        if n == "gate.weight":
            torch.testing.assert_close(eager_grads[n].float(), p.grad.float(), rtol=2e-2, atol=2e-2 * float(p.grad.float().abs().max()))
        else:
            assert torch.equal(eager_grads[n], p.grad), n
    torch.testing.assert_close(xe.grad.float(), xc.grad.float(), rtol=2e-2, atol=2e-2 * float(xc.grad.float().abs().max()))
