"""GPU parity for the reference's own expert-linear interface: Experts.forward in both call forms
(cute_kernels/kernels/scattermoe/torch_implementation.py:32-49; triton_implementation/__init__.py:14-36),
scattered_experts with the reference's argument list (triton_implementation/ops.py:295-316), the segment tables built
from a caller's sort, _compute_expert_assignment (torch_implementation.py:171-193), and a layer whose _compute_experts is
written the way the reference's MoE_Triton writes it.

Expected values are per-row fp32 / fp64 products written out here (no sort, no grouping); tolerances as in
test_gpu_moe.py (rtol 1e-2 / atol 1e-2 relative to each tensor's RMS for 16-bit results, 1e-4 for fp32).
"""

import numpy as np
import pytest
import torch
import torch.nn.functional as F

import cute_kernels
from cute_kernels import scattermoe
from oracle import integer_oracle as io
from test_gpu_moe import _run_layer_case

pytestmark = pytest.mark.gpu


def _close(ours, want, what, tol=1e-2, atol_factor=1.0):
    """Per element rtol = tol, atol = atol_factor * tol * RMS of the expected tensor (gradients pass 2 or 3, as the layer
    tests do: they are sums of rounded 16-bit terms); over the whole tensor an RMS error of at most tol / 2 of the RMS."""
    ours, want = ours.detach().double().cpu(), want.detach().double().cpu()
    rms = float(want.square().mean().sqrt())
    assert rms > 0.05, f"{what}: expected values too small to check ({rms})"
    torch.testing.assert_close(ours, want, rtol=tol, atol=atol_factor * tol * rms, msg=lambda m: f"{what}: {m}")
    assert float((ours - want).square().mean().sqrt()) <= 0.5 * tol * rms, what


def _routing(T, E, k, seed, device, empty=()):
    g = torch.Generator().manual_seed(seed)
    scores = torch.rand(T, E, generator=g)
    for e in empty:
        scores[:, e] = -1.0
    selected = scores.topk(k, dim=-1).indices  # k distinct experts per token
    flat = selected.flatten().to(device)
    sorted_expert_idxs, sorted_scattered_idxs = flat.sort(stable=True)  # what the reference's layer computes (int64)
    expert_offsets = flat.bincount(minlength=E).cumsum(-1)
    return selected, sorted_expert_idxs, sorted_scattered_idxs, expert_offsets


@pytest.mark.parametrize("idx_dtype", [torch.int64, torch.int32])
@pytest.mark.parametrize("T,E,k,align", [(300, 5, 2, 128), (4096, 8, 2, 256), (1000, 64, 8, 128), (7, 3, 1, 256)])
def test_segments_from_sorted_match_the_library_sort(device, idx_dtype, T, E, k, align):
    """Bit-exact: the tables derived from torch.sort + bincount + cumsum equal the ones ck_sort_by_expert derives from the
    unsorted ids (whose own parity against the C oracle is in test_gpu_routing.py), and row_pos is the sorted position."""
    selected, se, ss, off = _routing(T, E, k, 3, device, empty=(1,) if E > 2 else ())
    seg = cute_kernels.segments_from_sorted(se.to(idx_dtype), ss.to(idx_dtype), off.to(idx_dtype), align)
    ref = cute_kernels.sort_by_expert(selected.flatten().to(device), E, align)
    assert seg.max_rows == ref.max_rows and seg.align == align
    assert torch.equal(seg.seg_starts, ref.seg_starts) and torch.equal(seg.counts, ref.counts)
    assert torch.equal(seg.tile_expert, ref.tile_expert)
    starts, counts = ref.seg_starts.cpu().numpy(), ref.counts.cpu().numpy()
    first = np.concatenate([[0], np.cumsum(counts)[:-1]])
    slot, ref_slot, pos = seg.row_slot.cpu().numpy(), ref.row_slot.cpu().numpy(), seg.row_pos.cpu().numpy()
    for e in range(E):
        rows = slice(int(starts[e]), int(starts[e]) + int(counts[e]))
        assert np.array_equal(slot[rows], ref_slot[rows])
        assert np.array_equal(pos[rows], np.arange(first[e], first[e] + counts[e]))
    # and against the C oracle's stable sort of the same ids
    want_e, want_s = io.sort_by_expert(selected.flatten().numpy().astype(np.int32), E)
    assert np.array_equal(se.cpu().numpy(), want_e) and np.array_equal(ss.cpu().numpy(), want_s)


def _dense_expected(x_rows, w, row_expert, bias=None):
    """fp64: out[r] = w[expert of r] @ x_rows[r] (+ bias), row by row."""
    wr = w.double()[row_expert]  # [R, N, K]
    out = torch.einsum("rnk,rk->rn", wr, x_rows.double())
    if bias is not None:
        out = out + bias.double()[row_expert]
    return out


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("T,E,k,K,N", [(300, 5, 2, 128, 264), (3000, 4, 2, 256, 512), (257, 8, 4, 72, 64)])
@pytest.mark.parametrize("form", ["scatter", "grouped_out", "grouped_in", "grouped_in_out", "gated"])
@pytest.mark.parametrize("with_bias", [False, True])
def test_scattered_experts_forms(device, dtype, T, E, k, K, N, form, with_bias):
    """Forward and every gradient of one expert linear in each layout the reference's interface allows, against fp64
    autograd of the row-by-row definition."""
    tol = 1e-4 if dtype == torch.float32 else 1e-2
    selected, se, ss, off = _routing(T, E, k, 5, device, empty=(2,))
    g = torch.Generator().manual_seed(11)
    R = T * k
    grouped_in = form in ("grouped_in", "grouped_in_out", "gated")
    grouped_out = form in ("grouped_out", "grouped_in_out")
    w = (torch.randn(E, N, K, generator=g) * K**-0.5).to(dtype)
    bias = (0.3 * torch.randn(E, N, generator=g)).to(dtype) if with_bias else None
    x = torch.randn(R if grouped_in else T, K, generator=g).to(dtype)
    gates = torch.softmax(torch.randn(T, k, generator=g), dim=-1).to(dtype) if form == "gated" else None
    r_shape = (T, N) if form == "gated" else (R, N)
    cot = torch.randn(r_shape, generator=g).to(dtype)

    # ours
    xg = x.clone().to(device).requires_grad_()
    wg = w.clone().to(device).requires_grad_()
    bg = bias.clone().to(device).requires_grad_() if with_bias else None
    gg = gates.clone().to(device).requires_grad_() if gates is not None else None
    k_arg = 1 if grouped_in else k  # the reference's c_proj call passes 1 for grouped input
    out = cute_kernels.scattered_experts(xg, wg.permute(0, 2, 1), k_arg, se, ss, off, gg, grouped_in, grouped_out, bias=bg)
    assert out.shape == r_shape and out.dtype == dtype
    (out * cot.to(device)).sum().backward()

    # expected, in fp64, from the definition: sorted position p holds (token, slot) index ss[p] of expert se[p]
    se_c, ss_c = se.cpu(), ss.cpu()
    xe = x.double().requires_grad_()
    we = w.double().requires_grad_()
    be = bias.double().requires_grad_() if with_bias else None
    ge = gates.double().requires_grad_() if gates is not None else None
    rows_sorted = xe if grouped_in else xe[ss_c // k]  # input row of every sorted position
    y_sorted = _dense_expected(rows_sorted, we, se_c, be)  # [R, N] in sorted order
    if grouped_out:
        want = y_sorted
    else:
        y_slots = torch.zeros(R, N, dtype=torch.float64).index_put((ss_c,), y_sorted)  # back to (token, slot) order
        want = (ge.unsqueeze(-1) * y_slots.view(T, k, N)).sum(1) if ge is not None else y_slots
    (want * cot.double()).sum().backward()

    _close(out, want, f"{form} output", tol)
    _close(xg.grad, xe.grad, f"{form} input grad", tol, 2.0)
    mask = torch.zeros(E, dtype=torch.bool)
    mask[se_c.unique()] = True
    assert float(wg.grad[~mask.to(device)].abs().max()) == 0.0  # experts without rows: exact zeros (ops.py:252)
    _close(wg.grad, we.grad, f"{form} weight grad", tol, 3.0)
    if with_bias:
        _close(bg.grad, be.grad, f"{form} bias grad", tol, 3.0)
    if gates is not None:
        _close(gg.grad, ge.grad, f"{form} gate grad", tol, 3.0)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("add_bias", [False, True])
def test_experts_forward_with_expert_frequency(device, dtype, add_bias):
    """Experts_Torch.forward's form: grouped rows + per-expert counts in, F.linear per expert out; tensor or list input,
    tensor or list output; one expert without rows."""
    tol = 1e-4 if dtype == torch.float32 else 1e-2
    torch.manual_seed(0)
    E, K, N = 6, 128, 264
    layer = cute_kernels.Experts(E, K, N, add_bias=add_bias, std=K**-0.5).to(dtype).to(device)
    if add_bias:
        with torch.no_grad():
            layer.bias.normal_(0, 0.3)
    freq = torch.tensor([300, 0, 17, 520, 1, 64], device=device)
    x = torch.randn(int(freq.sum()), K, device=device, dtype=dtype)
    parts = x.split(freq.tolist())
    want = torch.cat([
        F.linear(parts[e].double(), layer.weight[e].double(), layer.bias[e].double() if add_bias else None) for e in range(E)
    ])
    out = layer(x, freq, return_list=False)
    _close(out, want, "tensor in, tensor out", tol)
    out_list = layer(x, freq, True)
    assert isinstance(out_list, list) and [o.size(0) for o in out_list] == freq.tolist()
    assert torch.equal(torch.cat(out_list), out)
    out_from_list = layer(tuple(parts), expert_frequency=freq, return_list=False)
    assert torch.equal(out_from_list, out)
    # uint32 counts, as continuous_count_cute returns them
    assert torch.equal(layer(x, cute_kernels.continuous_count_cute(torch.repeat_interleave(torch.arange(E, device=device), freq).int(), E), False), out)


class _LayerWrittenLikeTheReference(cute_kernels.MoE):
    """_compute_experts as the reference's accelerated layer writes it (triton_implementation/__init__.py:79-103): sort,
    offsets, c_fc(..., grouped_out=True), activation on the grouped rows, c_proj(..., 1, ..., grouped_in=True, gates=...)."""

    def _compute_experts(self, hidden_states, router_weights, selected_experts):
        sorted_expert_idxs, sorted_scattered_idxs = selected_experts.flatten().sort()
        expert_offsets = scattermoe.bincount(sorted_expert_idxs, self.num_experts).cumsum(-1)
        hidden_states = self.c_fc(
            hidden_states, self.top_k, sorted_expert_idxs, sorted_scattered_idxs, expert_offsets, grouped_out=True
        )
        hidden_states = self.act(hidden_states)
        hidden_states = self.c_proj(
            hidden_states, 1, sorted_expert_idxs, sorted_scattered_idxs, expert_offsets, grouped_in=True, gates=router_weights
        )
        return hidden_states


class _LayerWrittenLikeTheTorchReference(cute_kernels.MoE):
    """_compute_experts as the reference's torch layer writes it (torch_implementation.py:137-169), on this build's
    _compute_expert_assignment and Experts.forward(input, expert_frequency, return_list)."""

    def _compute_experts(self, hidden_states, router_weights, selected_experts):
        total_q = hidden_states.shape[0]
        fan_in_index, batch_gates, expert_frequency = self._compute_expert_assignment(router_weights, selected_experts)
        hidden_states = hidden_states[fan_in_index]
        hidden_states = self.c_fc(hidden_states, expert_frequency, return_list=True)
        hidden_states = [self.act(i) for i in hidden_states]
        hidden_states = self.c_proj(hidden_states, expert_frequency, return_list=False)
        # the gated sum over a token's k rows in fp32 (the reference's torch layer sums in the activation dtype with
        # index_add, whose order of additions on a GPU is not fixed: k roundings in an arbitrary order would need a
        # looser bound than the one this test shares with the other layer tests)
        weighted = hidden_states.float() * batch_gates.float().unsqueeze(-1)
        zeros = torch.zeros((total_q, self.hidden_size), dtype=torch.float32, device=hidden_states.device)
        return zeros.index_add(0, fan_in_index, weighted).to(hidden_states.dtype)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("act", ["swiglu", "glu", "gelu"])
@pytest.mark.parametrize("T,E,k,H,I", [(257, 8, 2, 128, 256), (700, 64, 8, 128, 136), (3000, 4, 2, 128, 256), (1, 6, 2, 256, 64)])
@pytest.mark.parametrize("layer_cls", [_LayerWrittenLikeTheReference, _LayerWrittenLikeTheTorchReference])
def test_layer_subclassed_the_reference_way_matches_the_oracle(device, dtype, act, T, E, k, H, I, layer_cls):
    # the torch-style layer gathers token rows with torch indexing, whose backward sums a token's k gradient rows in the
    # activation dtype in no fixed order (k roundings): x.grad gets twice the absolute bound there, everything else the same
    x_grad_atol = 4e-2 if layer_cls is _LayerWrittenLikeTheTorchReference else 2e-2
    _run_layer_case(device, dtype, T, E, k, H, I, act, moe_cls=layer_cls, x_grad_atol=x_grad_atol)


def test_layer_subclassed_the_reference_way_with_biases(device):
    _run_layer_case(device, torch.bfloat16, 3000, 4, 2, 128, 256, "gelu", add_bias=True, moe_cls=_LayerWrittenLikeTheReference)
    _run_layer_case(device, torch.bfloat16, 300, 4, 2, 128, 256, "glu", add_bias=True, moe_cls=_LayerWrittenLikeTheTorchReference,
                    x_grad_atol=4e-2)


def test_compute_expert_assignment(device):
    """Bit-exact against the C oracle's stable sort and histogram; the gates follow the permutation."""
    T, E, k = 1000, 16, 4
    moe = cute_kernels.MoE(E, k, 64, 72, cute_kernels.swiglu_packed_cute, True, False, 0.02)
    g = torch.Generator().manual_seed(2)
    selected = torch.rand(T, E, generator=g).topk(k, dim=-1).indices
    weights = torch.rand(T, k, generator=g).to(torch.bfloat16)
    fan_in, batch_gates, freq = moe._compute_expert_assignment(weights.to(device), selected.to(device))
    ids = selected.flatten().numpy().astype(np.int32)
    want_e, want_s = io.sort_by_expert(ids, E)
    assert np.array_equal(fan_in.cpu().numpy(), want_s // k)
    assert np.array_equal(freq.cpu().numpy(), io.count(ids, E)) and freq.dtype == torch.int64
    assert torch.equal(batch_gates.cpu(), weights.flatten()[torch.from_numpy(want_s.astype(np.int64))])


def test_no_tokens(device):
    """Zero tokens (an empty micro-batch) pass through the reference interface and the layer: empty results of the right
    shapes, zero gradients, no launch on NULL pointers."""
    E, K, N, k = 4, 64, 128, 2
    w1 = torch.randn(E, N, K, device=device, dtype=torch.bfloat16, requires_grad=True)
    w2 = torch.randn(E, K, N, device=device, dtype=torch.bfloat16, requires_grad=True)
    sel = torch.zeros(0, k, device=device, dtype=torch.long)
    se, ss = sel.flatten().sort(stable=True)
    off = scattermoe.bincount(se, E).cumsum(-1)
    assert off.tolist() == [0] * E
    x = torch.randn(0, K, device=device, dtype=torch.bfloat16, requires_grad=True)
    gates = torch.zeros(0, k, device=device, dtype=torch.bfloat16, requires_grad=True)
    h = cute_kernels.scattered_experts(x, w1.permute(0, 2, 1), k, se, ss, off, None, False, True)
    assert h.shape == (0, N)
    y = cute_kernels.scattered_experts(h, w2.permute(0, 2, 1), 1, se, ss, off, gates, True, False)
    assert y.shape == (0, K)
    y.sum().backward()
    assert x.grad.shape == (0, K) and gates.grad.shape == (0, k)
    assert float(w1.grad.abs().sum()) == 0.0 and float(w2.grad.abs().sum()) == 0.0

    layer = cute_kernels.MoE(E, k, K, N, cute_kernels.swiglu_packed_cute, True, False, 0.02).to(torch.bfloat16).to(device)
    x = torch.randn(2, 0, K, device=device, dtype=torch.bfloat16, requires_grad=True)
    out, logits = layer(x)
    assert out.shape == (2, 0, K) and logits.shape == (0, E)
    out.sum().backward()
    assert x.grad.shape == (2, 0, K)
    norm_weight = torch.ones(K, device=device, dtype=torch.bfloat16)
    out, logits = layer.forward_with_norm(x, norm_weight, 1e-5)
    assert out.shape == (2, 0, K) and logits.shape == (0, E)
