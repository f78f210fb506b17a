"""GPU parity for row movement (gather / combine / padded grouping / transposes), SwiGLU and RMSNorm against the torch
restatement in oracle/moe_oracle.py. Tolerances are the reference tests' own (swiglu_test.py:23-72,
rmsnorm_test.py:27-78) unless noted."""

import numpy as np
import pytest
import torch

import cute_kernels
from cute_kernels import _C, scattermoe
from oracle import moe_oracle as mo

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
def test_gather_rows_is_exact(device, dtype):
    g = torch.Generator().manual_seed(0)
    T, k, H = 300, 4, 96
    src = torch.randn(T, H, generator=g).to(dtype)
    idx = torch.randperm(T * k, generator=g).to(torch.int32)
    out = cute_kernels.gather_rows(src.to(device), idx.to(device), None, k)
    assert torch.equal(out.cpu(), src[(idx // k).long()])
    coeff = torch.rand(T * k, generator=g).to(dtype)
    out = cute_kernels.gather_rows(src.to(device), idx.to(device), coeff.to(device), k)
    expect = (src[(idx // k).long()].float() * coeff[idx.long()].float().unsqueeze(-1)).to(dtype)
    assert torch.equal(out.cpu(), expect)  # one fp32 multiply, one rounding: bit-exact


@pytest.mark.parametrize("dtype,tol", [(torch.bfloat16, 1e-2), (torch.float16, 2e-3), (torch.float32, 1e-5)])
def test_combine_rows_and_gate_grad(device, dtype, tol):
    g = torch.Generator().manual_seed(1)
    T, k, H = 257, 4, 128
    expanded = torch.randn(T, k, H, generator=g).to(dtype)
    gates = torch.rand(T, k, generator=g).to(dtype)
    grad_out = torch.randn(T, H, generator=g).to(dtype)
    out, _ = scattermoe._combine(expanded.to(device), gates.to(device), T, k, H)
    ref = torch.bmm(gates.float().unsqueeze(1), expanded.float()).squeeze(1)  # ops.py:173-174 in fp32
    torch.testing.assert_close(out.float().cpu(), ref, rtol=tol, atol=tol)
    summed, _ = scattermoe._combine(expanded.to(device), None, T, k, H)
    torch.testing.assert_close(summed.float().cpu(), expanded.float().sum(1), rtol=tol, atol=tol)  # ops.py:273-276
    _, dg = scattermoe._combine(expanded.to(device), None, T, k, H, grad_out=grad_out.to(device), want_out=False, want_d_gates=True)
    ref_dg = torch.bmm(expanded.float(), grad_out.float().unsqueeze(2)).squeeze(-1)  # ops.py:214
    torch.testing.assert_close(dg.float().cpu(), ref_dg, rtol=tol, atol=tol * 10)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("align", [128, 256])
def test_group_rows_padded_and_transposes(device, dtype, align):
    g = torch.Generator().manual_seed(2)
    T, k, H, E = 500, 2, 200, 5
    ids = torch.randint(0, E, (T * k,), generator=g, dtype=torch.int32)
    ids[ids == 3] = 1  # expert 3 is empty
    seg = cute_kernels.sort_by_expert(ids.to(device), E, align)
    src = torch.randn(T, H, generator=g).to(dtype)
    coeff = torch.rand(T * k, generator=g).to(dtype)
    grouped, grouped_t = scattermoe._group_rows(src.to(device), coeff.to(device), k, seg, True, True)
    seg_starts = seg.seg_starts.cpu().numpy()
    counts = seg.counts.cpu().numpy()
    row_slot = seg.row_slot.cpu().numpy()
    live = int(seg_starts[E])
    expect = torch.zeros(seg.max_rows, H, dtype=dtype)
    for e in range(E):
        for j in range(int(counts[e])):
            p = int(seg_starts[e]) + j
            slot = int(row_slot[p])
            expect[p] = (src[slot // k].float() * coeff[slot].float()).to(dtype)
    assert torch.equal(grouped.cpu()[:live], expect[:live])  # pad rows of live tiles are zero
    assert torch.equal(grouped_t.cpu()[:, :live], expect[:live].t())
    # without a transposed copy the whole-row kernel runs: same rows, same zero pad rows, identity mode too
    only_rows, none_t = scattermoe._group_rows(src.to(device), coeff.to(device), k, seg, True, False)
    assert none_t is None and torch.equal(only_rows.cpu()[:live], expect[:live])
    no_coeff, _ = scattermoe._group_rows(src.to(device), None, k, seg, True, False)
    tiled_no_coeff, _ = scattermoe._group_rows(src.to(device), None, k, seg, True, True)
    assert torch.equal(no_coeff.cpu()[:live], tiled_no_coeff.cpu()[:live])
    same, _ = scattermoe._group_rows(grouped, None, 0, seg, True, False)
    assert torch.equal(same.cpu()[:live], expect[:live])
    # identity mode (source already padded-grouped) and the batched weight transpose
    _, again_t = scattermoe._group_rows(grouped, None, 0, seg, False, True)
    assert torch.equal(again_t.cpu()[:, :live], expect[:live].t())
    w = torch.randn(3, 72, 40, generator=g).to(dtype)
    assert torch.equal(scattermoe._transpose_weights(w.to(device)).cpu(), w.transpose(1, 2).contiguous())


def _sizes_2d():
    sizes = [(2**i + j, 2**i + j) for i in range(0, 12, 2) for j in (0, 1, 7)]
    sizes += [(2999, 3001), (4096, 4096), (1, 8), (3, 1)]
    return sizes


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
def test_swiglu_reference_grid(device, dtype):
    g = torch.Generator().manual_seed(3)
    for size in _sizes_2d():
        gate = torch.randn(size, generator=g).to(dtype)
        up = torch.randn(size, generator=g).to(dtype)
        a, b = gate.clone().to(device).requires_grad_(), up.clone().to(device).requires_grad_()
        c, d = gate.clone().requires_grad_(), up.clone().requires_grad_()
        z = cute_kernels.swiglu_cute(a, b, kernel_backend_forward=None, kernel_backend_backward=None)
        z_ref = mo.swiglu_torch(c, d)
        z.mean().backward()
        z_ref.mean().backward()
        kw = dict(rtol=0, atol=5.5e-6) if dtype == torch.float32 else {}
        torch.testing.assert_close(z.cpu(), z_ref, **kw)
        kw = dict(rtol=0, atol=5e-6) if dtype == torch.float32 else {}
        torch.testing.assert_close(a.grad.cpu(), c.grad, **kw)
        torch.testing.assert_close(b.grad.cpu(), d.grad, **kw)


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
def test_swiglu_packed_reference_grid(device, dtype):
    g = torch.Generator().manual_seed(4)
    for size in _sizes_2d():
        size = (size[0], (size[1] + 1) // 2 * 2)
        x = torch.randn(size, generator=g).to(dtype)
        a, c = x.clone().to(device).requires_grad_(), x.clone().requires_grad_()
        z, z_ref = cute_kernels.swiglu_packed_cute(a), mo.swiglu_packed_torch(c)
        assert z.shape == (size[0], size[1] // 2)
        z.mean().backward()
        z_ref.mean().backward()
        kw = dict(rtol=0, atol=5.5e-6) if dtype == torch.float32 else {}
        torch.testing.assert_close(z.cpu(), z_ref, **kw)
        torch.testing.assert_close(a.grad.cpu(), c.grad, **(dict(rtol=0, atol=5e-6) if dtype == torch.float32 else {}))


def _rms_sizes():
    ns = sorted({2**i + j for i in range(0, 14, 2) for j in (0, 1, 5)} | {2048, 4096, 8192, 3001, 16384})
    out = []
    for n in ns:
        out += [(n,), (400, n)]
    return out


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
@pytest.mark.parametrize("has_weight", [True, False])
@pytest.mark.parametrize("memory_efficient", [True, False])
def test_rmsnorm_reference_grid(device, dtype, has_weight, memory_efficient):
    # reference grid rmsnorm_test.py:27-78 (which skips bf16; added here with bf16-sized bounds)
    g = torch.Generator().manual_seed(42)
    eps = 1e-5
    for size in _rms_sizes():
        x = torch.randn(size, generator=g).to(dtype)
        w = torch.randn(size[-1], generator=g).to(dtype) if has_weight else None
        a, c = x.clone().to(device).requires_grad_(), x.clone().requires_grad_()
        wa = w.clone().to(device).requires_grad_() if has_weight else None
        wc = w.clone().requires_grad_() if has_weight else None
        z = cute_kernels.rmsnorm_cute(x=a, weight=wa, eps=eps, memory_efficient=memory_efficient)
        z_ref = mo.rmsnorm_torch(c, wc, eps)
        z.sum().backward()
        z_ref.sum().backward()
        if dtype == torch.float32:
            torch.testing.assert_close(z.cpu(), z_ref, rtol=1.3e-6, atol=1e-5)
            torch.testing.assert_close(a.grad.cpu(), c.grad, rtol=1e-4, atol=1e-4)
            if has_weight:
                torch.testing.assert_close(wa.grad.cpu(), wc.grad, rtol=1e-4, atol=2e-4 * max(1, size[0] if len(size) > 1 else 1) ** 0.5)
        else:
            atol_z, atol_x = (1.6e-2, 9e-2) if dtype == torch.float16 else (6.3e-2, 0.36)
            torch.testing.assert_close(z.cpu(), z_ref, rtol=0, atol=atol_z)
            torch.testing.assert_close(a.grad.cpu(), c.grad, rtol=0, atol=atol_x)
            if has_weight:
                rt, at = (0.01, 0.1) if dtype == torch.float16 else (0.04, 0.5)
                torch.testing.assert_close(wa.grad.cpu(), wc.grad, rtol=rt, atol=at)


def test_rmsnorm_bf16_is_bit_exact_with_f_rms_norm_on_c4_rows(device):
    # F.rms_norm multiplies by the weight in fp32 and rounds once; so does the kernel
    g = torch.Generator().manual_seed(0)
    x = torch.randn(1024, 2048, generator=g).to(torch.bfloat16)
    w = (1 + 0.02 * torch.randn(2048, generator=g)).to(torch.bfloat16)
    z = cute_kernels.rmsnorm_cute(x.to(device), w.to(device), 1e-6)
    z_ref = mo.rmsnorm_torch(x, w, 1e-6)
    mismatch = (z.cpu() != z_ref).float().mean().item()
    assert mismatch < 2e-3, mismatch  # rsqrt / summation-order differences flip at most a few roundings
    torch.testing.assert_close(z.cpu().float(), z_ref.float(), rtol=1e-2, atol=1e-2)
    assert cute_kernels.rmsnorm_cute(x.to(device), None, None).dtype == torch.bfloat16


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("has_weight", [True, False])
@pytest.mark.parametrize("memory_efficient", [True, False])
@pytest.mark.parametrize("multiplier", [None, 0.9])
def test_fused_residual_add_rmsnorm_reference_grid(device, dtype, has_weight, memory_efficient, multiplier):
    # reference grid fused_residual_add_rmsnorm_test.py:20-90 (fp32 there; bf16 added with bf16-sized bounds)
    g = torch.Generator().manual_seed(42)
    eps = 1e-5
    for size in _rms_sizes():
        x = torch.randn(size, generator=g).to(dtype)
        r = torch.randn(size, generator=g).to(dtype)
        w = torch.randn(size[-1], generator=g).to(dtype) if has_weight else None
        xa, xc = x.clone().to(device).requires_grad_(), x.clone().requires_grad_()
        ra, rc = r.clone().to(device).requires_grad_(), r.clone().requires_grad_()
        wa = w.clone().to(device).requires_grad_() if has_weight else None
        wc = w.clone().requires_grad_() if has_weight else None
        z, added = cute_kernels.fused_residual_add_rmsnorm_cute(
            x=xa, residual=ra, weight=wa, eps=eps, multiplier=multiplier, memory_efficient=memory_efficient
        )
        z_ref, added_ref = mo.fused_residual_add_rmsnorm_torch(xc, rc, wc, eps, multiplier)
        # both outputs carry gradient, as in a transformer layer (the reference test does z * 2 + r * 3)
        (z.float() * 2 + added.float() * 3).sum().backward()
        (z_ref.float() * 2 + added_ref.float() * 3).sum().backward()
        assert torch.equal(added.cpu(), added_ref)  # the residual stream is bit-exact: same roundings
        if dtype == torch.float32:
            torch.testing.assert_close(z.cpu(), z_ref, rtol=1.3e-6, atol=1e-5)
            torch.testing.assert_close(xa.grad.cpu(), xc.grad, rtol=1e-4, atol=2e-4)
            torch.testing.assert_close(ra.grad.cpu(), rc.grad, rtol=1e-4, atol=2e-4)
            if has_weight:
                torch.testing.assert_close(wa.grad.cpu(), wc.grad, rtol=1e-4, atol=4e-4 * max(1, size[0] if len(size) > 1 else 1) ** 0.5)
        else:
            torch.testing.assert_close(z.cpu(), z_ref, rtol=0, atol=6.3e-2)
            torch.testing.assert_close(xa.grad.cpu(), xc.grad, rtol=2e-2, atol=0.72)
            torch.testing.assert_close(ra.grad.cpu(), rc.grad, rtol=2e-2, atol=0.72)
            if has_weight:
                torch.testing.assert_close(wa.grad.cpu(), wc.grad, rtol=0.04, atol=1.0)


def test_fused_residual_add_rmsnorm_without_residual_gradient(device):
    # only the normalised output is used downstream: the residual-stream gradient is absent (None -> zeros)
    g = torch.Generator().manual_seed(3)
    x, r = torch.randn(64, 512, generator=g), torch.randn(64, 512, generator=g)
    w = torch.randn(512, generator=g)
    xa, ra, wa = (t.clone().to(device).requires_grad_() for t in (x, r, w))
    xc, rc, wc = (t.clone().requires_grad_() for t in (x, r, w))
    z, _ = cute_kernels.fused_residual_add_rmsnorm_cute(xa, ra, wa, 1e-6, 0.5)
    z_ref, _ = mo.fused_residual_add_rmsnorm_torch(xc, rc, wc, 1e-6, 0.5)
    z.square().sum().backward()
    z_ref.square().sum().backward()
    for ours, ref in ((xa, xc), (ra, rc), (wa, wc)):
        torch.testing.assert_close(ours.grad.cpu(), ref.grad, rtol=1e-4, atol=1e-3)


def test_fused_residual_add_rmsnorm_backward_into_one_buffer(device):
    # multiplier 1: d_x and d_residual are the same values, and the C ABI takes one buffer for both (one store per row):
    # bit-identical to the two-buffer call; any other multiplier with one buffer is refused. Through autograd the two
    # leaves still end up with gradients of their own (a second backward accumulates into each separately).
    from cute_kernels import _C

    lib, stream = _C.lib(), torch.cuda.current_stream().cuda_stream
    g = torch.Generator().manual_seed(5)
    for B, H in ((300, 4096), (64, 512), (17, 8192)):
        added, d_out, d_added = (torch.randn(B, H, generator=g).to(torch.bfloat16).to(device) for _ in range(3))
        w = torch.randn(H, generator=g).to(torch.bfloat16).to(device)
        rstd = added.float().square().mean(-1).add(1e-6).rsqrt()
        partial = torch.empty(max(lib.ck_rmsnorm_bwd_partial_rows(B), 1), H, device=device, dtype=torch.float32)
        outs = []
        for one_buffer in (False, True):
            d_x, d_w = torch.empty_like(added), torch.empty(H, device=device, dtype=torch.float32)
            d_r = d_x if one_buffer else torch.empty_like(added)
            _C.check(lib.ck_fused_residual_add_rmsnorm_bwd(
                added.data_ptr(), w.data_ptr(), d_out.data_ptr(), d_added.data_ptr(), rstd.data_ptr(), 1e-6, 1.0, B, H,
                d_x.data_ptr(), d_r.data_ptr(), partial.data_ptr(), d_w.data_ptr(), _C.CK_BF16, stream))
            outs.append((d_x, d_r, d_w))
        assert torch.equal(outs[0][0], outs[0][1]) and torch.equal(outs[0][0], outs[1][0]) and torch.equal(outs[0][2], outs[1][2])
        d_x = torch.empty_like(added)
        with pytest.raises(RuntimeError, match="one buffer"):
            _C.check(lib.ck_fused_residual_add_rmsnorm_bwd(
                added.data_ptr(), w.data_ptr(), d_out.data_ptr(), d_added.data_ptr(), rstd.data_ptr(), 1e-6, 0.5, B, H,
                d_x.data_ptr(), d_x.data_ptr(), partial.data_ptr(), d_w.data_ptr(), _C.CK_BF16, stream))

    x, r = (torch.randn(64, 512, generator=g).to(device).requires_grad_() for _ in range(2))
    w = torch.randn(512, generator=g).to(device).requires_grad_()
    for _ in range(2):  # the second pass accumulates
        z, added = cute_kernels.fused_residual_add_rmsnorm_cute(x, r, w, 1e-6)
        (z * 2 + added * 3).sum().backward()
    assert x.grad.data_ptr() != r.grad.data_ptr() and torch.equal(x.grad, r.grad)
    xc, rc, wc = (t.detach().cpu().clone().requires_grad_() for t in (x, r, w))
    z_ref, added_ref = mo.fused_residual_add_rmsnorm_torch(xc, rc, wc, 1e-6, None)
    (z_ref * 2 + added_ref * 3).sum().backward()
    torch.testing.assert_close(x.grad.cpu(), 2 * xc.grad, rtol=1e-4, atol=4e-4)
    torch.testing.assert_close(w.grad.cpu(), 2 * wc.grad, rtol=1e-4, atol=4e-3)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("logits_multiplier", [None, 0.7])
def test_softmax_reference_grid(device, dtype, logits_multiplier):
    # reference grid and bounds: softmax_test.py:19-70 (std 0.02 inputs, sum().backward(), atol 4e-5 / 1.1e-3 on the grads)
    g = torch.Generator().manual_seed(42)
    for size in _rms_sizes() + [(3, 70000)]:
        x = (0.02 * torch.randn(size, generator=g)).to(dtype)
        a, c = x.clone().to(device).requires_grad_(), x.clone().requires_grad_()
        z = cute_kernels.softmax_cute(a, logits_multiplier)
        z_ref = mo.softmax_torch(c, logits_multiplier)
        z.sum().backward()
        z_ref.sum().backward()
        assert z.dtype == dtype and z.shape == x.shape
        if dtype == torch.float32:
            torch.testing.assert_close(z.cpu(), z_ref, rtol=1e-5, atol=1e-7)
            torch.testing.assert_close(a.grad.cpu(), c.grad, rtol=0, atol=4e-5)
        else:
            torch.testing.assert_close(z.cpu(), z_ref, rtol=1.6e-2, atol=1e-5)
            torch.testing.assert_close(a.grad.cpu(), c.grad, rtol=0, atol=1.1e-3)


def test_softmax_router_logits_shape_and_sharp_rows(device):
    # what a load-balancing loss does with the router logits the MoE layer returns: softmax over E, mean over tokens
    g = torch.Generator().manual_seed(1)
    logits = (4 * torch.randn(16384, 64, generator=g)).to(torch.bfloat16)
    p = cute_kernels.softmax_cute(logits.to(device))
    torch.testing.assert_close(p.float().cpu(), mo.softmax_torch(logits).float(), rtol=1.6e-2, atol=1e-6)
    # large-magnitude rows (max subtraction) and a weighted backward
    x = torch.randn(33, 4096, generator=g) * 30
    w = torch.randn(33, 4096, generator=g)
    a, c = x.clone().to(device).requires_grad_(), x.clone().requires_grad_()
    (cute_kernels.softmax_cute(a, 0.5) * w.to(device)).sum().backward()
    (mo.softmax_torch(c, 0.5) * w).sum().backward()
    torch.testing.assert_close(a.grad.cpu(), c.grad, rtol=1e-4, atol=1e-6)
