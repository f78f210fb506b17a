"""GPU parity (through the C ABI) for the integer stages: histogram/offsets, top-k routing, stable sort by expert.
Bit-exact against oracle/ck_oracle.c and against the committed fixtures."""

import os

import numpy as np
import pytest
import torch

import cute_kernels
from cute_kernels import _C
from oracle import integer_oracle as io

pytestmark = pytest.mark.gpu

GOLDEN = np.load(os.path.join(os.path.dirname(__file__), "golden", "routing_fixtures.npz"))


def _count_sizes():
    sizes = set()
    for i in range(15):  # the reference's 1-D size grid (tests/test_commons.py:30-40), thinned on j
        for j in (0, 1, 3, 7, 9):
            sizes.add(2**i + j)
    rng = np.random.default_rng(0)
    sizes.update(int(v) for v in rng.integers(2000, 4000, size=6))
    return sorted(sizes)


@pytest.mark.parametrize("dtype", [torch.int32, torch.long])
def test_continuous_count_reference_grid(device, dtype):
    # continuous_count_test.py:19-41 of the reference: ids ~ randint(0, 72), exact match with bincount
    g = torch.Generator().manual_seed(42)
    for n in _count_sizes():
        x = torch.randint(0, 72, (n,), generator=g, dtype=dtype)
        got = cute_kernels.continuous_count_cute(x.to(device), 72)
        assert got.dtype == torch.uint32 and got.shape == (72,)
        np.testing.assert_array_equal(got.cpu().numpy(), io.count(x.numpy(), 72), err_msg=f"n={n}")


@pytest.mark.parametrize("bins", [2, 8, 9, 16, 17, 64, 1000, 1024, 1025, 16384])
@pytest.mark.parametrize("dtype", [torch.int32, torch.long])
def test_count_offsets_bin_ranges(device, bins, dtype):
    g = torch.Generator().manual_seed(bins)
    for n in (0, 5, 70001, 1 << 20):
        x = torch.randint(0, bins, (n,), generator=g, dtype=dtype)
        counts, ends, starts = cute_kernels.continuous_count_and_offsets_cute(x.to(device), bins)
        c = io.count(x.numpy(), bins)
        e, s = io.offsets(c)
        np.testing.assert_array_equal(counts.cpu().numpy(), c)
        np.testing.assert_array_equal(ends.cpu().numpy(), e)
        np.testing.assert_array_equal(starts.cpu().numpy(), s)


def test_count_golden_c1_and_repeat_calls(device):
    ids = np.random.default_rng(int(GOLDEN["c1_seed"][0])).integers(0, 64, size=65536, dtype=np.int64)
    x = torch.from_numpy(ids).to(torch.int32).to(device)
    for _ in range(3):  # the workspace must come back to zero after every call
        counts, ends, starts = cute_kernels.continuous_count_and_offsets_cute(x, 64)
        np.testing.assert_array_equal(counts.cpu().numpy(), GOLDEN["c1_counts"])
        np.testing.assert_array_equal(ends.cpu().numpy(), GOLDEN["c1_ends"])
        np.testing.assert_array_equal(starts.cpu().numpy(), GOLDEN["c1_starts"])


def test_count_misaligned_views_out_of_range_and_shortcut(device):
    g = torch.Generator().manual_seed(5)
    base = torch.randint(-3, 80, (100003,), generator=g, dtype=torch.int32)
    for off in (1, 2, 3):
        x = base[off:]
        got = cute_kernels.continuous_count_cute(x.to(device)[0:], 72)  # keep the odd start through a device slice
        xd = base.to(device)[off:]
        got = cute_kernels.continuous_count_cute(xd, 72)
        np.testing.assert_array_equal(got.cpu().numpy(), io.count(x.numpy(), 72))
    out = cute_kernels.continuous_count_cute(torch.zeros(7, 3, device=device), 1)
    assert out.tolist() == [21] and out.dtype == torch.uint32
    strided = torch.arange(0, 64, dtype=torch.long, device=device).repeat(4)[::2]
    np.testing.assert_array_equal(
        cute_kernels.continuous_count_cute(strided, 64).cpu().numpy(), io.count(strided.cpu().numpy(), 64)
    )


def test_count_large_sum_property(device):
    # full-size property at 2^28 ids (1 GiB): counts sum to N and match a strided sample's histogram scaled check
    n = 1 << 28
    x = torch.randint(0, 64, (n,), dtype=torch.int32, device=device)
    counts, ends, starts = cute_kernels.continuous_count_and_offsets_cute(x, 64)
    c = counts.cpu().numpy().astype(np.int64)
    assert int(c.sum()) == n and int(ends[-1]) == n and int(starts[0]) == 0
    np.testing.assert_array_equal(c, torch.bincount(x, minlength=64).cpu().numpy())


@pytest.mark.parametrize("T,E,k", [(16384, 64, 2), (1000, 8, 2), (777, 8, 1), (513, 128, 8), (300, 6, 4), (64, 1000, 32), (5, 3, 3), (129, 72, 7)])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32, torch.float16])
def test_route_topk_softmax_matches_oracle(device, T, E, k, dtype):
    g = torch.Generator().manual_seed(42)
    logits = torch.randn(T, E, generator=g).to(dtype)  # bf16 rounding makes ties common (about 3% of C2 rows)
    sel, gates, vals = cute_kernels.route_topk_softmax_raw(logits.to(device), k)
    o_sel, o_gates, o_vals = io.topk_softmax(logits.float().numpy(), k)
    np.testing.assert_array_equal(sel.cpu().numpy(), o_sel)  # bit-exact, ties included (lowest index first)
    np.testing.assert_array_equal(vals.float().cpu().numpy(), o_vals)
    np.testing.assert_allclose(gates.cpu().numpy(), o_gates, rtol=2e-6, atol=1e-7)
    # and against torch.topk where it is defined: the values
    np.testing.assert_array_equal(vals.float().cpu().numpy(), logits.float().topk(k, dim=-1).values.numpy())


def test_route_special_values(device):
    row = torch.tensor([[1.0, 3.0, 3.0, -0.0, 0.0, 3.0, float("nan"), 2.0]])
    sel, _, _ = cute_kernels.route_topk_softmax_raw(row.to(device), 5)
    assert sel.tolist() == [[6, 1, 2, 5, 7]]
    sel, _, _ = cute_kernels.route_topk_softmax_raw(torch.tensor([[0.0, -0.0, -0.0, 0.0]], device=device), 4)
    assert sel.tolist() == [[0, 1, 2, 3]]


def test_route_autograd_matches_torch(device):
    g = torch.Generator().manual_seed(1)
    logits = torch.randn(257, 16, generator=g)  # fp32, no ties
    a = logits.clone().to(device).requires_grad_()
    b = logits.clone().requires_grad_()
    gates, sel = cute_kernels.route_topk_softmax(a, 4)
    v, i = b.topk(4, dim=-1)
    ref = torch.softmax(v.float(), dim=-1)
    assert sel.dtype == torch.long and torch.equal(sel.cpu(), i)
    w = torch.randn(257, 4, generator=g)
    (gates * w.to(device)).sum().backward()
    (ref * w).sum().backward()
    torch.testing.assert_close(gates.cpu(), ref, rtol=2e-6, atol=1e-7)
    torch.testing.assert_close(a.grad.cpu(), b.grad, rtol=1e-5, atol=1e-7)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_route_backward_takes_the_unrounded_gate_gradient_where_it_arrived_rounded(device, dtype):
    """ck_route_topk_softmax_bwd_exact against ck_route_topk_softmax_bwd fed with the gradient it has to pick: the fp32
    d_gates where the 16-bit gradient that arrived is that value rounded, the arrived value elsewhere (here every third
    row was doubled on its way, as a hook on the gates would). Bit-exact: same kernel arithmetic on the same inputs."""
    from cute_kernels import _C

    T, E, k = 777, 24, 4
    g = torch.Generator().manual_seed(5)
    logits = torch.randn(T, E, generator=g).to(dtype).to(device)
    sel, gates, _ = cute_kernels.route_topk_softmax_raw(logits, k)
    exact = torch.randn(T, k, generator=g).to(device)
    arrived = exact.to(dtype)
    arrived[::3] *= 2
    picked = torch.where(exact.to(dtype) == arrived, exact, arrived.float())
    assert 0 < int((picked != exact).sum()) < T * k
    lib = _C.lib()
    got = torch.full((T, E), 7.0, dtype=dtype, device=device)
    want = torch.full((T, E), 9.0, dtype=dtype, device=device)
    with torch.cuda.device(device):
        _C.check(lib.ck_route_topk_softmax_bwd_exact(_C.ptr(gates), _C.ptr(exact), _C.ptr(arrived), _C.ptr(sel), T, E, k,
                                                     _C.ptr(got), _C.dtype_code(dtype), _C.stream()))
        _C.check(lib.ck_route_topk_softmax_bwd(_C.ptr(gates), _C.ptr(picked), _C.ptr(sel), T, E, k, _C.ptr(want),
                                               _C.dtype_code(dtype), _C.stream()))
    assert torch.equal(got, want)
    # against autograd of softmax over the selected logits with the picked gradient
    v = torch.gather(logits.float(), 1, sel.long()).requires_grad_()
    torch.softmax(v, -1).backward(picked)
    ref = torch.zeros(T, E, device=device).scatter_(1, sel.long(), v.grad)
    torch.testing.assert_close(got.float(), ref, rtol=1e-2, atol=1e-3)
    rc = lib.ck_route_topk_softmax_bwd_exact(_C.ptr(gates), _C.ptr(exact), _C.ptr(exact), _C.ptr(sel), T, E, k, _C.ptr(got),
                                             _C.CK_F32, _C.stream())
    assert rc != 0  # fp32 gradients have nothing to recover


def _check_sort(device, ids: torch.Tensor, E: int, align: int):
    seg = cute_kernels.sort_by_expert(ids.to(device), E, align)
    idn = ids.numpy().astype(np.int64)
    se, ss = io.sort_by_expert(idn, E)
    c = io.count(idn, E)
    e, s = io.offsets(c)
    np.testing.assert_array_equal(seg.sorted_expert_idxs.cpu().numpy(), se)
    np.testing.assert_array_equal(seg.sorted_scattered_idxs.cpu().numpy(), ss)
    np.testing.assert_array_equal(seg.counts.cpu().numpy(), c)
    np.testing.assert_array_equal(seg.ends.cpu().numpy(), e)
    np.testing.assert_array_equal(seg.starts.cpu().numpy(), s)
    o_seg_starts, o_row_slot, o_tile = io.segments(c, ss, align, seg.max_rows)
    np.testing.assert_array_equal(seg.seg_starts.cpu().numpy(), o_seg_starts)
    np.testing.assert_array_equal(seg.tile_expert.cpu().numpy()[: seg.max_rows // align], o_tile)
    got_slot = seg.row_slot.cpu().numpy()[: seg.max_rows]
    valid = o_row_slot >= 0  # pad rows are left unwritten by the kernel
    np.testing.assert_array_equal(got_slot[valid], o_row_slot[valid])
    return seg


@pytest.mark.parametrize("R,E", [(32768, 64), (32768, 8), (65536, 64), (524288, 128), (1, 128), (2, 2), (1000, 1), (4097, 72), (8, 4096),
                                  (65537, 64), (100000, 8), (40000, 800), (40000, 900)])
@pytest.mark.parametrize("align", [128, 256])
@pytest.mark.parametrize("dtype", [torch.int32, torch.long])
def test_sort_by_expert_matches_oracle(device, R, E, align, dtype):
    g = torch.Generator().manual_seed(R + E)
    ids = torch.randint(0, E, (R,), generator=g, dtype=dtype)
    _check_sort(device, ids, E, align)


def test_sort_empty_experts_zipf_and_golden(device):
    ids = torch.from_numpy(GOLDEN["small_ids"])
    E = int(GOLDEN["small_num_experts"][0])
    seg = _check_sort(device, ids, E, 128)
    np.testing.assert_array_equal(seg.sorted_scattered_idxs.cpu().numpy(), GOLDEN["small_sorted_scattered_idxs"])
    np.testing.assert_array_equal(seg.sorted_expert_idxs.cpu().numpy(), GOLDEN["small_sorted_expert_idxs"])
    # Zipf(1.0)-like load over 8 experts, the C3 routing shape
    p = 1.0 / np.arange(1, 9)
    ids = torch.from_numpy(np.random.default_rng(0).choice(8, size=32768, p=p / p.sum()))
    for _ in range(2):  # second call reuses the self-restoring workspace
        _check_sort(device, ids, 8, 256)
    # all rows to one expert, at the far end
    _check_sort(device, torch.full((5000,), 63, dtype=torch.int32), 64, 128)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("T,E,k", [(16384, 64, 2), (1000, 128, 8), (1, 8, 2)])
def test_load_balancing_loss_matches_oracle(device, dtype, T, E, k):
    """cute_kernels.load_balancing_loss (continuous_count_cute + softmax_cute) against the one-hot formulation in the
    oracle: value and gradient w.r.t. the router logits. fp32 1e-5; bf16: the probabilities are rounded to bf16 before
    the mean (rtol 1e-2)."""
    from oracle import moe_oracle as mo

    g = torch.Generator().manual_seed(E + k)
    logits = torch.randn(T, E, generator=g).to(dtype)
    sel = torch.stack([torch.randperm(E, generator=g)[:k] for _ in range(min(T, 64))])
    sel = sel.repeat((T + sel.size(0) - 1) // sel.size(0), 1)[:T]
    lg = logits.clone().to(device).requires_grad_()
    loss = cute_kernels.load_balancing_loss(lg, sel.to(device))
    loss.backward()
    lo = logits.clone().float().requires_grad_()
    want = mo.load_balancing_loss_torch(lo, sel)
    want.backward()
    tol = dict(rtol=1e-5, atol=1e-6) if dtype == torch.float32 else dict(rtol=1e-2, atol=1e-3)
    torch.testing.assert_close(loss.cpu(), want.detach(), **tol)
    gtol = dict(rtol=1e-4, atol=1e-7) if dtype == torch.float32 else dict(rtol=5e-2, atol=2e-4 / max(T, 1) + 1e-6)
    torch.testing.assert_close(lg.grad.float().cpu(), lo.grad, **gtol)
    f, P = cute_kernels.load_balancing_stats(lg.detach(), sel.to(device))
    assert abs(float(f.sum()) - k) < 1e-5 and abs(float(P.sum()) - 1.0) < 1e-2


def test_sort_by_expert_out_of_range_ids_are_dropped_and_can_be_detected(device):
    """The contract for ids outside [0, E): dropped from counts and offsets (ends[-1] < R), the rest sorted as if they
    were not there; validate=True turns that into an error."""
    ids = torch.tensor([3, 0, 7, 2, 2, -1, 1, 0, 9, 3], dtype=torch.int32)
    E = 4
    seg = cute_kernels.sort_by_expert(ids.to(device), E, 128)
    keep = (ids >= 0) & (ids < E)
    want_counts = torch.bincount(ids[keep].long(), minlength=E)
    assert seg.counts.cpu().long().tolist() == want_counts.tolist()
    placed = int(seg.ends[-1])
    assert placed == int(keep.sum()) < ids.numel()
    order = [i for e in range(E) for i in range(ids.numel()) if int(ids[i]) == e]  # stable sort of the valid ids
    assert seg.sorted_scattered_idxs[:placed].cpu().tolist() == order
    assert seg.sorted_expert_idxs[:placed].cpu().tolist() == sorted(ids[keep].tolist())
    with pytest.raises(ValueError, match="outside"):
        cute_kernels.sort_by_expert(ids.to(device), E, 128, validate=True)
    cute_kernels.sort_by_expert(ids[keep].to(device), E, 128, validate=True)  # all in range: no error
