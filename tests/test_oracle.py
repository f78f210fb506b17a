"""Pins the CPU oracle (oracle/) before anything is compared against it.

Each oracle function is checked against something that is NOT its own formula: a numpy/torch library routine, brute
force on tiny inputs, an independent dense formulation in fp64, invariants, and the committed fixtures in tests/golden.
"""

import os

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from oracle import integer_oracle as io
from oracle import moe_oracle as mo

GOLDEN = np.load(os.path.join(os.path.dirname(__file__), "golden", "routing_fixtures.npz"))


# ---- integer stages ------------------------------------------------------------------------------------------
@pytest.mark.parametrize("n,bins", [(0, 5), (1, 1), (7, 3), (1000, 72), (65536, 64), (4099, 16384)])
def test_count_matches_bincount_and_brute_force(n, bins):
    rng = np.random.default_rng(n + bins)
    ids = rng.integers(0, bins, size=n, dtype=np.int64)
    got = io.count(ids, bins)
    assert got.dtype == np.uint32
    np.testing.assert_array_equal(got, np.bincount(ids, minlength=bins))
    if n <= 1000:
        brute = [sum(1 for v in ids if v == e) for e in range(bins)]
        np.testing.assert_array_equal(got, brute)
    assert int(got.sum()) == n


def test_count_ignores_out_of_range():
    ids = np.array([-1, 0, 3, 3, 4, 100, 2**40], dtype=np.int64)
    np.testing.assert_array_equal(io.count(ids, 4), [1, 0, 0, 2])


def test_count_golden_c1():
    ids = np.random.default_rng(int(GOLDEN["c1_seed"][0])).integers(0, 64, size=65536, dtype=np.int64)
    counts = io.count(ids, 64)
    np.testing.assert_array_equal(counts, GOLDEN["c1_counts"])
    ends, starts = io.offsets(counts)
    np.testing.assert_array_equal(ends, GOLDEN["c1_ends"])
    np.testing.assert_array_equal(starts, GOLDEN["c1_starts"])


def test_offsets_match_cumsum():
    counts = np.random.default_rng(0).integers(0, 1000, size=129).astype(np.uint32)
    ends, starts = io.offsets(counts)
    np.testing.assert_array_equal(ends, np.cumsum(counts))
    np.testing.assert_array_equal(starts, np.cumsum(counts) - counts)
    assert ends[-1] == counts.sum() and starts[0] == 0
    assert np.all(np.diff(ends.astype(np.int64)) >= 0)


@pytest.mark.parametrize("n,E", [(0, 4), (1, 1), (50, 3), (32768, 8), (65536, 64), (5000, 128)])
def test_sort_matches_stable_argsort(n, E):
    rng = np.random.default_rng(n * 31 + E)
    ids = rng.integers(0, E, size=n, dtype=np.int64)
    se, ss = io.sort_by_expert(ids, E)
    order = np.argsort(ids, kind="stable")
    np.testing.assert_array_equal(ss, order)
    np.testing.assert_array_equal(se, ids[order])
    t_sorted, t_order = torch.sort(torch.from_numpy(ids), stable=True)
    np.testing.assert_array_equal(ss, t_order.numpy())
    np.testing.assert_array_equal(se, t_sorted.numpy())
    # invariants: a permutation, keys non-decreasing, positions increasing inside each expert
    assert sorted(ss.tolist()) == list(range(n))
    assert np.all(np.diff(se) >= 0)
    same = np.diff(se) == 0
    assert np.all(np.diff(ss)[same] > 0)


def test_sort_golden_small():
    ids = GOLDEN["small_ids"]
    E = int(GOLDEN["small_num_experts"][0])
    se, ss = io.sort_by_expert(ids, E)
    np.testing.assert_array_equal(se, GOLDEN["small_sorted_expert_idxs"])
    np.testing.assert_array_equal(ss, GOLDEN["small_sorted_scattered_idxs"])
    np.testing.assert_array_equal(io.count(ids, E), GOLDEN["small_counts"])


@pytest.mark.parametrize("align", [1, 4, 128])
def test_segments_brute_force(align):
    rng = np.random.default_rng(align)
    E = 6
    ids = rng.choice(np.array([0, 1, 3, 5]), size=37).astype(np.int64)  # experts 2 and 4 are empty
    counts = io.count(ids, E)
    _, ss = io.sort_by_expert(ids, E)
    max_rows = -(-(ids.size + E * (align - 1)) // align) * align
    seg_starts, row_slot, tile_expert = io.segments(counts, ss, align, max_rows)
    # brute force, expert by expert
    run = 0
    for e in range(E):
        assert seg_starts[e] == run and run % align == 0
        members = [i for i in range(ids.size) if ids[i] == e]  # already in increasing order = stable order
        assert row_slot[run : run + len(members)].tolist() == members
        padded = -(-len(members) // align) * align
        assert np.all(row_slot[run + len(members) : run + padded] == -1)
        assert np.all(tile_expert[run // align : (run + padded) // align] == e)
        run += padded
    assert seg_starts[E] == run
    assert np.all(tile_expert[run // align :] == -1)
    assert np.all(row_slot[run:] == -1)


# ---- routing -------------------------------------------------------------------------------------------------
def test_topk_values_and_non_tie_indices_match_torch_topk():
    torch.manual_seed(0)
    logits = torch.randn(2048, 64).to(torch.bfloat16).float()
    k = 2
    sel, gates, vals = io.topk_softmax(logits.numpy(), k)
    t_vals, t_idx = logits.topk(k, dim=-1)
    np.testing.assert_array_equal(vals, t_vals.numpy())  # values are unique whatever the tie order
    srt = torch.sort(logits, dim=-1, descending=True).values
    tie_rows = (srt[:, k - 1] == srt[:, k]) | (srt[:, 0] == srt[:, 1])
    assert tie_rows.any() and not tie_rows.all()  # bf16-rounded logits do tie
    np.testing.assert_array_equal(sel[~tie_rows.numpy()], t_idx.numpy()[~tie_rows.numpy()])
    # tie rows: still a valid selection of the right values, without repeats
    picked = np.take_along_axis(logits.numpy(), sel.astype(np.int64), axis=1)
    np.testing.assert_array_equal(picked, vals)
    assert all(len(set(r)) == k for r in sel.tolist())
    # agrees with the stable descending sort (the tie rule, via a library routine)
    o_vals, o_idx = mo.topk_lowest_index_first(logits, k)
    np.testing.assert_array_equal(sel, o_idx.numpy())
    np.testing.assert_array_equal(vals, o_vals.numpy())


def test_topk_tie_rule_and_special_values():
    row = np.array([[1.0, 3.0, 3.0, -0.0, 0.0, 3.0, np.nan, 2.0]], dtype=np.float32)
    sel, gates, vals = io.topk_softmax(row, 5)
    assert sel.tolist() == [[6, 1, 2, 5, 7]]  # NaN first (torch order), then equal 3.0s by index
    sel, _, _ = io.topk_softmax(np.array([[0.0, -0.0, -0.0, 0.0]], dtype=np.float32), 4)
    assert sel.tolist() == [[0, 1, 2, 3]]  # signed zeros tie


def test_topk_gates_are_softmax_of_selected():
    rng = np.random.default_rng(3)
    logits = rng.standard_normal((257, 40)).astype(np.float32)
    sel, gates, vals = io.topk_softmax(logits, 8)
    expect = torch.softmax(torch.from_numpy(vals), dim=-1).numpy()
    np.testing.assert_allclose(gates, expect, rtol=1e-6, atol=1e-7)
    np.testing.assert_allclose(gates.sum(-1), 1.0, rtol=1e-6)
    # equivalent to softmax over all experts, top-k, renormalise
    full = torch.softmax(torch.from_numpy(logits).double(), dim=-1)
    top = full.gather(-1, torch.from_numpy(sel.astype(np.int64)))
    np.testing.assert_allclose(gates, (top / top.sum(-1, keepdim=True)).numpy(), rtol=1e-5)


# ---- floating-point stages -------------------------------------------------------------------------------------
def test_swiglu_closed_form_and_packed_order():
    torch.manual_seed(1)
    gate, up = torch.randn(33, 17, dtype=torch.float64), torch.randn(33, 17, dtype=torch.float64)
    expect = up * gate / (1 + torch.exp(-gate))
    # the reference computes in fp32 whatever the input dtype (.float(), swiglu/torch_implementation.py:11-12)
    torch.testing.assert_close(mo.swiglu_torch(gate, up), expect, rtol=2e-6, atol=2e-6)
    # packed: FIRST half is up, SECOND half is gate (reference swiglu/__init__.py:121)
    torch.testing.assert_close(mo.swiglu_packed_torch(torch.cat([up, gate], -1)), expect, rtol=2e-6, atol=2e-6)
    assert not torch.allclose(mo.swiglu_packed_torch(torch.cat([gate, up], -1)), expect)


def test_rmsnorm_closed_form_and_gradcheck():
    torch.manual_seed(2)
    x = torch.randn(5, 24, dtype=torch.float64, requires_grad=True)
    w = torch.randn(24, dtype=torch.float64, requires_grad=True)
    eps = 1e-5
    expect = x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps) * w
    torch.testing.assert_close(mo.rmsnorm_torch(x, w, eps), expect, rtol=1e-12, atol=1e-12)
    assert torch.autograd.gradcheck(lambda a, b: mo.rmsnorm_torch(a, b, eps), (x, w))
    # backward closed form of the reference README (rmsnorm/README.md:27-29)
    dy = torch.randn(5, 24, dtype=torch.float64)
    (gx,) = torch.autograd.grad(mo.rmsnorm_torch(x, w, eps), x, dy)
    rstd = 1 / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)
    expect_gx = rstd * dy * w - x * rstd**3 / 24 * (dy * w * x).sum(-1, keepdim=True)
    torch.testing.assert_close(gx, expect_gx, rtol=1e-10, atol=1e-12)
    assert mo.rmsnorm_torch(x.detach().float(), None, None).dtype == torch.float32


def _dense_moe_fp64(moe: mo.MoEOracle, x: torch.Tensor) -> torch.Tensor:
    """Independent formulation: per token, loop over its k experts; no sort, no bincount, no index_add."""
    xd = x.double()
    logits = xd @ moe.gate.weight.double().t()
    out = torch.zeros_like(xd)
    for t in range(xd.size(0)):
        order = sorted(range(moe.num_experts), key=lambda e: (-float(logits[t, e]), e))[: moe.top_k]
        v = torch.stack([logits[t, e] for e in order])
        g = torch.exp(v - v.max())
        g = g / g.sum()
        for j, e in enumerate(order):
            h = moe.c_fc.weight[e].double() @ xd[t]
            h = moe.act(h)
            out[t] += g[j] * (moe.c_proj.weight[e].double() @ h)
    return out


@pytest.mark.parametrize("is_glu", [True, False])
@pytest.mark.parametrize("E,k", [(4, 2), (6, 4), (8, 1)])
def test_moe_oracle_matches_dense_per_token_formulation(E, k, is_glu):
    torch.manual_seed(E * 10 + k)
    def glu64(v):  # [up | gate] packed SwiGLU kept in fp64 (swiglu_packed_torch itself computes in fp32)
        up, gate = v.chunk(2, dim=-1)
        return up * F.silu(gate)

    act = glu64 if is_glu else torch.nn.GELU(approximate="tanh")
    moe = mo.MoEOracle(E, k, 16, 24, act, is_glu, False, 0.5).double()
    x = torch.randn(19, 16, dtype=torch.float64)
    y, logits = moe(x)
    # gates go through an fp32 softmax in the reference (torch_implementation.py:132), hence ~1e-7 relative noise;
    # a wrong index, sign or operand order would show up at O(1)
    torch.testing.assert_close(y, _dense_moe_fp64(moe, x), rtol=1e-5, atol=1e-5)
    torch.testing.assert_close(logits, x @ moe.gate.weight.t())
    assert y.shape == x.shape and logits.shape == (19, E)
    # leading dims are flattened and restored (torch_implementation.py:103-120)
    y3, _ = moe(x.view(1, 19, 16))
    torch.testing.assert_close(y3.view(19, 16), y)


def test_moe_oracle_state_dict_keys_and_shapes():
    moe = mo.MoEOracle(4, 2, 16, 24, mo.swiglu_packed_torch, True, False, 0.02)
    sd = moe.state_dict()
    assert list(sd) == ["gate.weight", "c_fc.weight", "c_proj.weight"]
    assert sd["gate.weight"].shape == (4, 16)
    assert sd["c_fc.weight"].shape == (4, 48, 16)  # 2*I rows when is_glu
    assert sd["c_proj.weight"].shape == (4, 16, 24)
    assert abs(float(sd["c_fc.weight"].std()) - 0.02) < 0.005


def test_fused_residual_add_rmsnorm_closed_form():
    g = torch.Generator().manual_seed(5)
    x, r = torch.randn(7, 33, generator=g, dtype=torch.float64), torch.randn(7, 33, generator=g, dtype=torch.float64)
    w = torch.randn(33, generator=g, dtype=torch.float64)
    for mult in (None, 1, 0.9):
        y, added = mo.fused_residual_add_rmsnorm_torch(x, r, w, 1e-5, mult)
        a = x * (1.0 if mult is None else mult) + r  # written out, not through the oracle
        torch.testing.assert_close(added, a, rtol=0, atol=0)
        expect = a / torch.sqrt((a * a).mean(-1, keepdim=True) + 1e-5) * w
        torch.testing.assert_close(y, expect, rtol=1e-12, atol=1e-12)
    # a dropped multiplier or a swapped operand would show: y depends on x only through mult * x + r
    y1, _ = mo.fused_residual_add_rmsnorm_torch(x, r, None, 1e-5, 0.5)
    y2, _ = mo.fused_residual_add_rmsnorm_torch(0.5 * x, r, None, 1e-5, None)
    torch.testing.assert_close(y1, y2, rtol=1e-12, atol=1e-12)
    # the 16-bit path rounds the scaled x and the sum separately
    xb, rb = x.to(torch.bfloat16), r.to(torch.bfloat16)
    _, added_b = mo.fused_residual_add_rmsnorm_torch(xb, rb, None, 1e-5, 0.9)
    assert torch.equal(added_b, ((xb.float() * 0.9).to(torch.bfloat16).float() + rb.float()).to(torch.bfloat16))


def test_softmax_closed_form_and_jacobian():
    g = torch.Generator().manual_seed(9)
    x = torch.randn(5, 17, generator=g, dtype=torch.float64, requires_grad=True)
    for mult in (None, 0.7):
        m = 1.0 if mult is None else mult
        y = mo.softmax_torch(x, mult)
        e = torch.exp(m * x.detach() - (m * x.detach()).amax(-1, keepdim=True))  # written out, not through F.softmax
        torch.testing.assert_close(y.detach().double(), e / e.sum(-1, keepdim=True), rtol=1e-6, atol=1e-7)  # fp32 inside
        assert torch.allclose(y.sum(-1).double(), torch.ones(5, dtype=torch.float64), atol=1e-6)
        # backward closed form: d_x = m * y * (d_y - sum(d_y * y)); a dropped multiplier or sign would show
        dy = torch.randn(5, 17, generator=g, dtype=torch.float64)
        (gx,) = torch.autograd.grad(y, x, dy.to(y.dtype))
        yd = y.detach().double()
        torch.testing.assert_close(gx, m * yd * (dy - (dy * yd).sum(-1, keepdim=True)), rtol=1e-5, atol=1e-6)
    assert mo.softmax_torch(x.detach().to(torch.bfloat16), 0.7).dtype == torch.bfloat16


def test_load_balancing_loss_closed_form_and_invariants():
    """The auxiliary-loss oracle against the formula written with counts (no one-hot): E * sum_e (count_e / T) * P_e; a
    perfectly balanced router gives k; a dropped factor E, a mean over the wrong axis or probabilities of the selected
    experts only would each fail one of these."""
    g = torch.Generator().manual_seed(11)
    T, E, k = 97, 8, 2
    logits = torch.randn(T, E, generator=g, dtype=torch.float64)
    sel = torch.stack([torch.randperm(E, generator=g)[:k] for _ in range(T)])
    counts = torch.bincount(sel.flatten(), minlength=E).double()
    e = torch.exp(logits - logits.amax(-1, keepdim=True))
    P = (e / e.sum(-1, keepdim=True)).mean(0)
    want = E * torch.sum(counts / T * P)
    torch.testing.assert_close(mo.load_balancing_loss_torch(logits, sel).double(), want, rtol=1e-6, atol=1e-7)
    # uniform logits and a round-robin assignment: f_e = k / E, P_e = 1 / E -> loss = k
    uniform = torch.zeros(96, E)
    sel_rr = (torch.arange(96 * k).reshape(96, k)) % E
    assert abs(float(mo.load_balancing_loss_torch(uniform, sel_rr)) - k) < 1e-6
    # everything routed to one expert that also has all the probability mass: loss = E * k
    peaked = torch.full((16, E), -1e4)
    peaked[:, 3] = 0.0
    assert abs(float(mo.load_balancing_loss_torch(peaked, torch.full((16, k), 3))) - E * k) < 1e-4


# ---- fp8 (e4m3fn) quantiser and quantised-expert forward ----------------------------------------------------------
def _e4m3fn_table() -> np.ndarray:
    """All 256 OCP e4m3fn values from the format definition (1 sign, 4 exponent bits with bias 7, 3 mantissa bits;
    exponent 0 is subnormal; S.1111.111 is NaN; there is no infinity), written out without any library cast."""
    vals = np.empty(256, dtype=np.float64)
    for code in range(256):
        sign = -1.0 if code & 0x80 else 1.0
        exp, man = (code >> 3) & 0xF, code & 0x7
        if exp == 0xF and man == 0x7:
            vals[code] = np.nan
        elif exp == 0:
            vals[code] = sign * (man / 8.0) * 2.0**-6
        else:
            vals[code] = sign * (1.0 + man / 8.0) * 2.0 ** (exp - 7)
    return vals


def _nearest_e4m3fn_code(v: float, table: np.ndarray) -> int:
    """Brute force: the finite code closest to v; on an exact tie the one with an even mantissa bit (even code)."""
    best, best_d = None, None
    for code in range(256):
        if np.isnan(table[code]) or (table[code] == 0 and code == 0x80 and not np.signbit(v)):
            continue
        if table[code] == 0 and code == 0x00 and np.signbit(v):
            continue
        d = abs(table[code] - v)
        if best is None or d < best_d or (d == best_d and code % 2 == 0 and best % 2 == 1):
            best, best_d = code, d
    return best


def _quantize_rows_brute(x64: np.ndarray, table: np.ndarray):
    """Independent per-row quantiser: scale = amax / 448 (1 for an all-zero row), q = nearest table value of
    fp32(x * fp32(448 / amax))."""
    codes = np.zeros(x64.shape, dtype=np.uint8)
    scales = np.ones(x64.shape[0], dtype=np.float32)
    for r in range(x64.shape[0]):
        row = x64[r].astype(np.float32)
        amax = np.float32(np.abs(row).max())
        inv = np.float32(1.0)
        if amax > 0:
            scales[r] = amax / np.float32(448.0)
            inv = np.float32(448.0) / amax
        for c in range(row.size):
            codes[r, c] = _nearest_e4m3fn_code(float(np.float32(row[c] * inv)), table)
    return codes, scales


def test_e4m3fn_table_facts():
    t = _e4m3fn_table()
    assert np.nanmax(t) == 448.0 and np.nanmin(t) == -448.0
    assert t[0x7E] == 448.0 and np.isnan(t[0x7F]) and np.isnan(t[0xFF])
    assert t[0x01] == 2.0**-9 and t[0x08] == 2.0**-6 and t[0x38] == 1.0  # smallest subnormal / normal, one
    assert np.sum(np.isfinite(t)) == 254
    # torch's cast decodes the same table (library routine against the format definition)
    decoded = torch.arange(256, dtype=torch.uint8).view(torch.float8_e4m3fn).float().numpy()
    np.testing.assert_array_equal(np.nan_to_num(decoded, nan=12345.0), np.nan_to_num(t, nan=12345.0).astype(np.float32))


def test_quantize_rows_e4m3_against_brute_force_nearest_value():
    table = _e4m3fn_table()
    g = torch.Generator().manual_seed(21)
    rows = [
        torch.randn(24, generator=g),                                  # ordinary row, maximum somewhere inside
        torch.zeros(24),                                               # all-zero row: scale 1, codes 0
        torch.tensor([0.1, -3.0, 0.2] + [0.0] * 21),                    # negative maximum, not at index 0
        torch.tensor([448.0] + [v for v in (17.0, 19.0, 21.0, 23.0, 25.0, 27.0, 29.0, 31.0)] + [0.0] * 15),  # ties: odd multiples of the half step in [16, 32)
        torch.tensor([448.0, 2.0**-9, 2.0**-10, 1.5 * 2.0**-10, 3.0 * 2.0**-10, 2.0**-7 + 2.0**-10] + [0.0] * 18),  # subnormals and their ties
        torch.tensor([1e-30, -1e-31] + [0.0] * 22),                     # tiny maximum: scale far below 1
        torch.tensor([3e38, -1e38, 5.0] + [0.0] * 21),                  # huge maximum
        torch.randn(24, generator=g) * 1e-3,
    ]
    x = torch.stack(rows)
    q, scale = mo.quantize_rows_e4m3_torch(x)
    assert q.dtype == torch.float8_e4m3fn and scale.dtype == torch.float32 and scale.shape == (len(rows),)
    codes, scales = _quantize_rows_brute(x.double().numpy(), table)
    got = q.view(torch.uint8).numpy()
    # +0 and -0 decode to the same value: compare decoded values, then codes where the value is not zero
    np.testing.assert_array_equal(table[got], table[codes])
    nz = table[codes] != 0
    np.testing.assert_array_equal(got[nz], codes[nz])
    np.testing.assert_array_equal(scale.numpy(), scales)
    # scale = amax / 448, and 1 for the all-zero row
    amax = x.abs().amax(-1)
    assert float(scale[1]) == 1.0 and not np.any(got[1] & 0x7F)
    np.testing.assert_array_equal(scale[amax > 0].numpy(), (amax[amax > 0] / 448.0).numpy())
    # the row maximum saturates exactly at +-448
    for r in range(len(rows)):
        if float(amax[r]) > 0:
            i = int(x[r].abs().argmax())
            assert table[got[r, i]] == (448.0 if float(x[r, i]) > 0 else -448.0)
    # ties go to the even mantissa: 17 -> 16, 19 -> 20, 21 -> 20, 23 -> 24, ... (step 2 in [16, 32))
    assert table[got[3, 1:9]].tolist() == [16.0, 20.0, 20.0, 24.0, 24.0, 28.0, 28.0, 32.0]
    # subnormals (step 2^-9): 2^-9 exact, 2^-10 ties to 0, 1.5 * 2^-10 rounds up to 2^-9, 3 * 2^-10 ties to 2^-8
    assert table[got[4, 1:5]].tolist() == [2.0**-9, 0.0, 2.0**-9, 2.0**-8]
    # the error bound of round-to-nearest: |x - q * scale| <= half a step of the binade of the scaled value
    deq = table[got] * scale.double().numpy()[:, None]
    scaled = np.abs(x.double().numpy() / scale.double().numpy()[:, None])
    step = np.where(scaled < 2.0**-6, 2.0**-9, 2.0 ** (np.floor(np.log2(np.maximum(scaled, 2.0**-6))) - 3))
    assert np.all(np.abs(x.double().numpy() - deq) <= (0.5 * step * (1 + 1e-6)) * scale.double().numpy()[:, None])


def test_quantize_rows_e4m3_scale_direction_and_dtypes():
    """De-quantisation is q * scale (not q / scale), whatever the input dtype; a swapped direction is off by (amax/448)^2."""
    table = _e4m3fn_table()
    for dtype in (torch.float32, torch.bfloat16, torch.float16):
        x = (torch.randn(5, 40, generator=torch.Generator().manual_seed(4)) * 7).to(dtype)
        q, s = mo.quantize_rows_e4m3_torch(x)
        deq = table[q.view(torch.uint8).numpy()] * s.double().numpy()[:, None]
        rel = np.linalg.norm(deq - x.double().numpy()) / np.linalg.norm(x.double().numpy())
        assert rel < 0.04  # 3 mantissa bits: about 2^-4 / sqrt(3) relative error per element


def _bf16(v: np.ndarray) -> np.ndarray:
    """fp64 -> nearest bfloat16 (ties to even) as fp64, through bit arithmetic on the fp32 pattern (no torch cast)."""
    f = np.asarray(v, dtype=np.float64).astype(np.float32)
    bits = f.view(np.uint32).astype(np.uint64)
    rounded = ((bits + 0x7FFF + ((bits >> 16) & 1)) >> 16) << 16
    return rounded.astype(np.uint32).view(np.float32).astype(np.float64)


def _dense_e4m3_moe_fp64(moe, x, selected, gates, table):
    """Independent formulation of the quantised-expert forward: brute-force quantiser, table de-quantisation, fp64
    products per token and slot, 16-bit roundings where a 16-bit tensor sits (pre-activation, activation, expert
    output, combined output). No call into oracle/."""
    E, H = moe.num_experts, x.shape[1]
    w1c, w1s = _quantize_rows_brute(moe.c_fc.weight.detach().double().flatten(0, 1).numpy(), table)
    w2c, w2s = _quantize_rows_brute(moe.c_proj.weight.detach().double().flatten(0, 1).numpy(), table)
    w1 = (table[w1c] * w1s.astype(np.float64)[:, None]).reshape(E, -1, H)
    w2 = (table[w2c] * w2s.astype(np.float64)[:, None]).reshape(E, H, -1)
    xc, xs = _quantize_rows_brute(x.double().numpy(), table)
    xd = table[xc] * xs.astype(np.float64)[:, None]
    I = w2.shape[2]
    out = np.zeros(x.shape, dtype=np.float64)
    for t in range(x.shape[0]):
        for j in range(selected.shape[1]):
            e = int(selected[t, j])
            pre = _bf16(w1[e] @ xd[t])
            up, gate = pre[:I], pre[I:]
            act = _bf16(up * gate / (1.0 + np.exp(-gate)))
            ac, a_s = _quantize_rows_brute(act[None], table)
            y = _bf16(w2[e] @ (table[ac[0]] * float(a_s[0])))
            out[t] += float(gates[t, j]) * y
    return _bf16(out)


def test_moe_e4m3_forward_oracle_matches_dense_fp64_formulation_on_table():
    table = _e4m3fn_table()
    torch.manual_seed(33)
    E, k, H, I, T = 4, 2, 32, 48, 9
    moe = mo.MoEOracle(E, k, H, I, mo.swiglu_packed_torch, True, False, 0.25).to(torch.bfloat16)
    x = torch.randn(T, H).to(torch.bfloat16)
    x[3] = 0  # an all-zero token: scale 1, output 0
    sel = torch.stack([torch.randperm(E)[:k] for _ in range(T)])
    gates = torch.softmax(torch.randn(T, k), -1).to(torch.bfloat16)
    got = mo.moe_e4m3_forward_oracle(moe, x, sel, gates).double().numpy()
    want = _dense_e4m3_moe_fp64(moe, x, sel.numpy(), gates.double().numpy(), table)
    assert np.abs(want).mean() > 0.05  # an O(0.1 .. 1) signal, so that the tolerance below means something
    assert not np.any(got[3]) and not np.any(want[3])
    # fp32 against fp64 accumulation can move a value across a bf16 rounding boundary now and then, and such a flip
    # can move an activation to the neighbouring e4m3 value: allow two bf16 steps, and require most elements bit-equal.
    # A mistake in the specification (scale direction, the zero-row rule, a missing 16-bit rounding of the
    # pre-activation or the activation, up/gate swapped, gates applied before the rounding of y) is far outside.
    np.testing.assert_allclose(got, want, rtol=2.0**-6, atol=2.0**-9)
    assert np.mean(got == want) > 0.9
    # sensitivity: with the up and gate halves of c_fc exchanged the result is nowhere near
    swapped = mo.MoEOracle(E, k, H, I, mo.swiglu_packed_torch, True, False, 0.25).to(torch.bfloat16)
    swapped.load_state_dict(moe.state_dict())
    with torch.no_grad():
        swapped.c_fc.weight.copy_(torch.cat(moe.c_fc.weight.chunk(2, dim=1)[::-1], dim=1))
    assert not np.allclose(mo.moe_e4m3_forward_oracle(swapped, x, sel, gates).double().numpy(), want, rtol=2.0**-6, atol=2.0**-9)
