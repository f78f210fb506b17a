"""GPU parity for the RMSNorm fused ahead of the router (ck_rmsnorm_route, through the C ABI): against the oracle
composition gate(rmsnorm(x)) -- rmsnorm/torch_implementation.py:9-10 and scattermoe/torch_implementation.py:122-124 of the
reference -- and against the library's own separate kernels.

Tolerances: y and logits rtol = atol = 1e-2 against the oracle (16-bit outputs); the logits additionally within one
rounding step of their dtype of the fp64 product of the kernel's own y with the gate weight (they are computed from that
y); rstd 1e-6 relative; e4m3 rows and scales bit-exact against the quantiser applied to the kernel's y."""

import pytest
import torch
import torch.nn.functional as F

import cute_kernels
from cute_kernels import rmsnorm_route
from oracle import moe_oracle as mo

pytestmark = pytest.mark.gpu


def _inputs(dtype, B, H, E, seed, with_weight=True):
    g = torch.Generator().manual_seed(seed)
    x = (torch.randn(B, H, generator=g) * (0.5 + 2 * torch.rand(B, 1, generator=g))).to(dtype)
    w = (1 + 0.1 * torch.randn(H, generator=g)).to(dtype) if with_weight else None
    gate = (torch.randn(E, H, generator=g) * H**-0.5).to(dtype)
    return x, w, gate


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize(
    "B,H,E,with_weight",
    [(16, 512, 16, True), (1, 512, 8, True), (37, 1024, 64, True), (300, 2048, 64, False), (129, 1536, 60, True),
     (1000, 4096, 128, True), (50, 3584, 100, False), (33, 2560, 1, True)],
)
def test_rmsnorm_route_matches_oracle_composition(device, dtype, B, H, E, with_weight):
    x, w, gate = _inputs(dtype, B, H, E, B + H + E, with_weight)
    eps = 1e-6
    assert rmsnorm_route.rmsnorm_route_fused(x, gate)
    y, logits, x8, scale8 = cute_kernels.rmsnorm_route_cute(
        x.to(device), None if w is None else w.to(device), gate.to(device), eps, quantize=True, fused=True
    )
    oracle_y = mo.rmsnorm_torch(x, w, eps)
    oracle_logits = F.linear(oracle_y.float(), gate.float())
    torch.testing.assert_close(y.cpu().float(), oracle_y.float(), rtol=1e-2, atol=1e-2)
    # the separate kernel computes the same expression with another summation order for rstd: at most one step apart
    y_sep = cute_kernels.rmsnorm_cute(x.to(device), None if w is None else w.to(device), eps)
    step = 2.0**-7 if dtype == torch.bfloat16 else 2.0**-10
    assert float(((y.float() - y_sep.float()).abs() / (y_sep.float().abs() + 1e-6)).max()) <= step
    assert float((y != y_sep).float().mean()) < 1e-3
    assert logits.shape == (B, E) and logits.dtype == dtype
    torch.testing.assert_close(logits.cpu().float(), oracle_logits, rtol=1e-2, atol=1e-2)
    own = y.cpu().double() @ gate.double().t()
    assert float(((logits.cpu().double() - own).abs() / (own.abs() + 1.0)).max()) <= step
    # e4m3 rows: exactly the quantiser applied to the stored y
    q_sep, s_sep = cute_kernels.quantize_rows_e4m3(y)
    assert torch.equal(x8.view(torch.uint8), q_sep.view(torch.uint8)) and torch.equal(scale8, s_sep)
    oq, os_ = mo.quantize_rows_e4m3_torch(y.cpu())
    assert torch.equal(x8.cpu().view(torch.uint8), oq.view(torch.uint8)) and torch.equal(scale8.cpu(), os_)


def test_rmsnorm_route_rstd_and_all_zero_rows(device):
    x, w, gate = _inputs(torch.bfloat16, 40, 1024, 32, 5)
    x[3] = 0
    eps = 1e-5
    from cute_kernels import _C

    xd, wd, gd = x.to(device), w.to(device), gate.to(device)
    y = torch.empty_like(xd)
    logits = torch.empty(40, 32, dtype=torch.bfloat16, device=device)
    rstd = torch.empty(40, dtype=torch.float32, device=device)
    ws = torch.empty(32 * 1024, dtype=torch.bfloat16, device=device)
    _C.check(_C.lib().ck_rmsnorm_route(_C.ptr(xd), _C.ptr(wd), _C.ptr(gd), eps, 40, 1024, 32, _C.ptr(y), _C.ptr(rstd),
                                       _C.ptr(logits), None, None, _C.ptr(ws), _C.dtype_code(torch.bfloat16), _C.stream()))
    want = torch.rsqrt(x.double().square().mean(-1) + eps)
    torch.testing.assert_close(rstd.cpu().double(), want, rtol=1e-6, atol=0)
    assert torch.all(y[3] == 0) and torch.all(logits[3] == 0)


def test_rmsnorm_route_rejects_unsupported_shapes_and_falls_back(device):
    from cute_kernels import _C

    t = torch.zeros(16, 640, dtype=torch.bfloat16, device=device)
    g = torch.zeros(8, 640, dtype=torch.bfloat16, device=device)
    out = torch.zeros(16, 8, dtype=torch.bfloat16, device=device)
    rc = _C.lib().ck_rmsnorm_route(_C.ptr(t), None, _C.ptr(g), 1e-6, 16, 640, 8, _C.ptr(t), None, _C.ptr(out), None, None,
                                   _C.ptr(t), _C.dtype_code(torch.bfloat16), _C.stream())
    assert rc != 0 and b"multiple of 512" in _C.lib().ck_last_error_string()
    # the Python entry point composes the separate kernels for such shapes
    x, w, gate = _inputs(torch.bfloat16, 20, 640, 8, 9)
    assert not rmsnorm_route.rmsnorm_route_fused(x, gate)
    y, logits = cute_kernels.rmsnorm_route_cute(x.to(device), w.to(device), gate.to(device), 1e-6)
    oracle_y = mo.rmsnorm_torch(x, w, 1e-6)
    torch.testing.assert_close(y.cpu().float(), oracle_y.float(), rtol=1e-2, atol=1e-2)
    torch.testing.assert_close(logits.cpu().float(), F.linear(oracle_y.float(), gate.float()), rtol=1e-2, atol=1e-2)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("with_weight", [True, False])
def test_rmsnorm_route_backward(device, dtype, with_weight):
    """Gradients of (x, norm weight, gate weight) for a loss that uses both outputs, against fp32 autograd of the oracle
    composition on the same 16-bit inputs; criterion relative to each gradient's RMS (2e-2: 16-bit outputs of sums)."""
    B, H, E = 200, 1024, 32
    x, w, gate = _inputs(dtype, B, H, E, 11, with_weight)
    g = torch.Generator().manual_seed(1)
    d_y = torch.randn(B, H, generator=g).to(dtype)
    d_logits = torch.randn(B, E, generator=g).to(dtype)
    leaves = [t.to(device).requires_grad_() for t in (x, gate)] + ([w.to(device).requires_grad_()] if with_weight else [])
    y, logits = cute_kernels.rmsnorm_route_cute(leaves[0], leaves[2] if with_weight else None, leaves[1], 1e-6)
    torch.autograd.backward([y, logits], [d_y.to(device), d_logits.to(device)])
    ref = [t.float().requires_grad_() for t in (x, gate)] + ([w.float().requires_grad_()] if with_weight else [])
    ry = mo.rmsnorm_torch(ref[0], ref[2] if with_weight else None, 1e-6)
    torch.autograd.backward([ry, F.linear(ry, ref[1])], [d_y.float(), d_logits.float()])
    for name, ours, truth in zip(("x", "gate", "norm weight"), leaves, ref):
        assert ours.grad.dtype == dtype
        scale = float(truth.grad.square().mean().sqrt())
        err = float((ours.grad.cpu().float() - truth.grad).abs().max())
        assert err <= 2e-2 * scale * 8, f"{name}: {err} against RMS {scale}"
        assert float((ours.grad.cpu().float() - truth.grad).square().mean().sqrt()) <= 1e-2 * scale, name


def test_moe_forward_with_norm_equals_norm_then_forward(device):
    """The module's fused-prologue entry: same selection (bit-exact top-k on its own logits), output and gradients as the
    layer applied to rmsnorm_cute(x)."""
    torch.manual_seed(2)
    T, H, E, k, I = 700, 1024, 16, 2, 512
    moe = cute_kernels.MoE(E, k, H, I, cute_kernels.swiglu_packed_cute, True, False, H**-0.5).to(torch.bfloat16).to(device)
    w = (1 + 0.1 * torch.randn(H, device=device)).to(torch.bfloat16)
    x = torch.randn(T, H, device=device, dtype=torch.bfloat16)
    xa, xb = x.clone().requires_grad_(), x.clone().requires_grad_()
    wa, wb = w.clone().requires_grad_(), w.clone().requires_grad_()
    ya, la = moe.forward_with_norm(xa, wa, 1e-6)
    # selection: the library's top-k on the fused logits against the oracle's rule on the same logits
    _, sel = cute_kernels.route_topk_softmax(la.detach(), k)
    _, want_sel = mo.topk_lowest_index_first(la.detach().cpu(), k)
    assert torch.equal(sel.cpu(), want_sel)
    go = torch.randn_like(ya)
    ya.backward(go)
    grads_a = {n: p.grad.clone() for n, p in moe.named_parameters()}
    for p in moe.parameters():
        p.grad = None
    yb, lb = moe(cute_kernels.rmsnorm_cute(xb, wb, 1e-6))
    yb.backward(go)
    torch.testing.assert_close(la.float(), lb.float(), rtol=1e-2, atol=1e-2)
    same = (cute_kernels.route_topk_softmax(lb.detach(), k)[1] == sel).all(dim=-1)
    assert float(same.float().mean()) > 0.98  # near-ties may flip with the logits' last bit
    torch.testing.assert_close(ya[same].float(), yb[same].float(), rtol=2e-2, atol=2e-2)

    def close(a, b, what):
        scale = float(b.float().square().mean().sqrt())
        assert float((a.float() - b.float()).square().mean().sqrt()) <= 5e-2 * scale, what

    close(xa.grad, xb.grad, "x.grad")
    close(wa.grad, wb.grad, "norm weight grad")
    for n, p in moe.named_parameters():
        close(grads_a[n], p.grad, n)


def test_moe_e4m3_forward_with_norm(device):
    torch.manual_seed(3)
    T, H, E, k, I = 600, 1024, 8, 2, 512
    moe = cute_kernels.MoE(E, k, H, I, cute_kernels.swiglu_packed_cute, True, False, H**-0.5).to(torch.bfloat16).to(device)
    q = cute_kernels.MoE_E4M3(moe)
    w = (1 + 0.1 * torch.randn(H, device=device)).to(torch.bfloat16)
    x = torch.randn(T, H, device=device, dtype=torch.bfloat16)
    ya, la = q.forward_with_norm(x, w, 1e-6)
    yb, lb = q(cute_kernels.rmsnorm_cute(x, w, 1e-6))
    torch.testing.assert_close(la.float(), lb.float(), rtol=1e-2, atol=1e-2)
    same = (cute_kernels.route_topk_softmax(lb, k)[1] == cute_kernels.route_topk_softmax(la, k)[1]).all(dim=-1)
    assert float(same.float().mean()) > 0.98
    torch.testing.assert_close(ya[same].float(), yb[same].float(), rtol=5e-2, atol=5e-2)
