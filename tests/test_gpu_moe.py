"""GPU parity for the scattered grouped GEMMs (every epilogue, through the C ABI) and for the whole MoE layer,
forward and backward, against the torch restatement of the reference (oracle/moe_oracle.py).

Tolerance for bf16 / fp16 results with fp32 accumulation: rtol 1e-2, atol 1e-2 against the oracle. Where the oracle's own
bf16 rounding is the larger error (its index_add combine sums in bf16, torch_implementation.py:163-165; weight grads
under a sum loss), the check goes through an fp32 run of the same oracle: |ours - truth| <= |oracle - truth| + tol.
"""

import numpy as np
import pytest
import torch
import torch.nn as nn
import torch.nn.functional as F

import cute_kernels
from cute_kernels import _C, scattermoe
from oracle import moe_oracle as mo

pytestmark = pytest.mark.gpu

RTOL, ATOL = 1e-2, 1e-2


def _layout(seg):
    return seg.seg_starts.cpu().numpy(), seg.counts.cpu().numpy(), seg.row_slot.cpu().numpy()


def _expected_grouped(a_rows_fn, w, seg, N):
    """fp32 reference of Y = A_e @ W[e]^T over the padded grouped layout (pad rows zero)."""
    seg_starts, counts, row_slot = _layout(seg)
    out = torch.zeros(seg.max_rows, N)
    for e in range(seg.num_experts):
        s, c = int(seg_starts[e]), int(counts[e])
        if c:
            rows = torch.stack([a_rows_fn(p, int(row_slot[p])) for p in range(s, s + c)]).float()
            out[s : s + c] = F.linear(rows, w[e].float())  # the per-expert loop of torch_implementation.py:39-44
    return out


@pytest.fixture(params=["default", "general"])
def gemm_tile(request):
    """Which kernel the 16-bit GEMMs run on: the library's own choice (the 128-byte-row kernel wherever it applies: align
    256 and K % 64 == 0), or the general kernel for every case (ck_debug_set_option "gemm_line_kernel")."""
    if request.param != "default":
        _C.set_option("gemm_line_kernel", 0)
    yield request.param
    _C.set_option("gemm_line_kernel", 1)


def _make_case(device, dtype, T, k, E, align, empty=(3,), seed=0):
    g = torch.Generator().manual_seed(seed)
    ids = torch.randint(0, E, (T * k,), generator=g, dtype=torch.int32)
    for e in empty:
        if e < E:
            ids[ids == e] = 0
    seg = cute_kernels.sort_by_expert(ids.to(device), E, align)
    return g, seg


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("align", [128, 256])
@pytest.mark.parametrize("K,N", [(200, 136), (64, 128), (576, 264), (160, 840), (192, 840), (320, 392)])
def test_grouped_gemm_gather_in_grouped_out(device, dtype, align, K, N, gemm_tile):
    T, k, E = 300, 2, 5
    g, seg = _make_case(device, dtype, T, k, E, align)
    x = torch.randn(T, K, generator=g).to(dtype)
    w = (0.1 * torch.randn(E, N, K, generator=g)).to(dtype)
    y = torch.zeros(seg.max_rows, N, dtype=dtype, device=device)
    y_t = torch.full((N, seg.ld_t), 7.0, dtype=dtype, device=device)
    scattermoe._gemm(x.to(device), k, w.to(device), seg, _C.CK_EPI_GROUPED, y, y_t=y_t)
    expect = _expected_grouped(lambda p, slot: x[slot // k], w, seg, N)
    live = int(seg.seg_starts[E])
    torch.testing.assert_close(y.float().cpu()[:live], expect[:live], rtol=RTOL, atol=ATOL)
    assert torch.equal(y_t.cpu()[:, :live], y.cpu()[:live].t())  # same roundings, zeros in pad rows


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("align", [128, 256])
@pytest.mark.parametrize("K,N", [(136, 200), (160, 840), (128, 840), (320, 264)])
def test_grouped_gemm_grouped_in_scatter_out(device, dtype, align, K, N, gemm_tile):
    T, k, E = 300, 2, 5
    g, seg = _make_case(device, dtype, T, k, E, align, seed=1)
    h = torch.randn(seg.max_rows, K, generator=g).to(dtype)
    w = (0.1 * torch.randn(E, N, K, generator=g)).to(dtype)
    y = torch.full((T * k, N), float("nan"), dtype=dtype, device=device)
    scattermoe._gemm(h.to(device), 0, w.to(device), seg, _C.CK_EPI_SCATTER, y)
    grouped = _expected_grouped(lambda p, slot: h[p], w, seg, N)
    seg_starts, counts, row_slot = _layout(seg)
    expect = torch.zeros(T * k, N)
    for e in range(E):
        for p in range(int(seg_starts[e]), int(seg_starts[e]) + int(counts[e])):
            expect[int(row_slot[p])] = grouped[p]
    assert not torch.isnan(y.float()).any()  # every (token, slot) row was written exactly once
    torch.testing.assert_close(y.float().cpu(), expect, rtol=RTOL, atol=ATOL)


@pytest.mark.parametrize("N", [5120, 6400, 7168])  # 13 row tiles x 20 / 25 / 28 column tiles: last round 4 / 69 / 108 tiles (4 / 3 / 2 parts)
@pytest.mark.parametrize("form", ["nt_grouped", "nt_scatter", "nn_grouped", "nn_scatter"])
def test_grouped_gemm_split_last_round(device, monkeypatch, form, N):
    """A launch whose last round of tiles is at most a quarter full computes those tiles in four parts of the contraction
    (ck_grouped_gemm_ws / ck_grouped_gemm_nn_ws with a workspace). Against the same launch without the workspace
    (scattermoe.options.gemm_split = False): equal up to the fp32 re-association of four partial sums (rtol = atol = 1e-2,
    and at least 99 % of the elements bit-equal); two split launches in a row are bit-identical (fixed order of additions),
    also when the arrival words at the end of the workspace hold leftovers of a launch that never finished (every bit
    pattern is "nobody has arrived yet" to a later launch); against the fp32 reference at the GEMM tolerance."""
    T, k, E, align = 1400, 2, 6, 256
    K = 2048
    g, seg = _make_case(device, torch.bfloat16, T, k, E, align, empty=(3,), seed=11)
    live_tiles = int(seg.seg_starts[E]) // align * (N // 256)
    assert 0 < live_tiles % 256 <= 128 and live_tiles // 256 <= 64, live_tiles  # the split applies to this launch
    scatter = form.endswith("scatter")
    rows_out = T * k if scatter else seg.max_rows
    epi = _C.CK_EPI_SCATTER if scatter else _C.CK_EPI_GROUPED
    if form.startswith("nt"):
        a = torch.randn(T, K, generator=g).to(torch.bfloat16).to(device)
        w = (torch.randn(E, N, K, generator=g) * K**-0.5).to(torch.bfloat16).to(device)
        run = lambda out: scattermoe._gemm(a, k, w, seg, epi, out)
    else:
        a = torch.randn(seg.max_rows, K, generator=g).to(torch.bfloat16).to(device)
        w = (torch.randn(E, K, N, generator=g) * K**-0.5).to(torch.bfloat16).to(device)  # [E, out = K here, in = N]
        run = lambda out: scattermoe._gemm_dx(a, w, seg, epi, out)
    outs = []
    ws = scattermoe._split_workspace(device)
    for split in (True, True, "dirty", False):
        monkeypatch.setattr(scattermoe.options, "gemm_split", bool(split))
        if split == "dirty":  # stale arrival words: counts in flight, another epoch, all ones
            words = ws[-512:].view(torch.int32)
            words[0::3] = 3
            words[1::3] = (12345 << 4) | 2
            words[2::3] = -1
        out = torch.zeros(rows_out, N, dtype=torch.bfloat16, device=device)
        run(out)
        outs.append(out)
    assert torch.equal(outs[0], outs[1]) and torch.equal(outs[0], outs.pop(2))
    torch.testing.assert_close(outs[0].float(), outs[2].float(), rtol=RTOL, atol=ATOL)
    assert float((outs[0] == outs[2]).float().mean()) > 0.99
    # fp32 reference on a sample of rows
    seg_starts, counts, row_slot = _layout(seg)
    checked = 0
    for e in range(E):
        s_, c_ = int(seg_starts[e]), int(counts[e])
        for p in list(range(s_, s_ + c_))[:: max(1, c_ // 5)][:6]:
            slot = int(row_slot[p])
            src = a[slot // k] if form.startswith("nt") else a[p]
            want = (src.float() @ (w[e].float().t() if form.startswith("nt") else w[e].float())).cpu()
            got = outs[0][slot if scatter else p].float().cpu()
            torch.testing.assert_close(got, want, rtol=RTOL, atol=ATOL)
            checked += 1
    assert checked > 10


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("with_bias", [False, True])
@pytest.mark.parametrize("align,K,N", [(128, 200, 136), (256, 64, 128), (256, 576, 264), (256, 192, 840)])
def test_grouped_gemm_gelu_tanh_epilogue(device, dtype, align, K, N, with_bias, gemm_tile):
    """CK_EPI_GELU_TANH: y as the grouped epilogue writes it (bias in the accumulators), and aux = the tanh GELU of the
    rounded y -- against torch's F.gelu(approximate="tanh") (the reference test's activation module, test_commons.py:85-86)
    applied to the kernel's own y (within one rounding step of the 16-bit type) and to the fp32 reference."""
    T, k, E = 300, 2, 5
    g, seg = _make_case(device, dtype, T, k, E, align, seed=3)
    x = torch.randn(T, K, generator=g).to(dtype)
    w = (0.1 * torch.randn(E, N, K, generator=g)).to(dtype)
    bias = torch.randn(E, N, generator=g).to(dtype) if with_bias else None
    y = torch.zeros(seg.max_rows, N, dtype=dtype, device=device)
    act = torch.full((seg.max_rows, N), 9.0, dtype=dtype, device=device)
    scattermoe._gemm(x.to(device), k, w.to(device), seg, _C.CK_EPI_GELU_TANH, y, aux=act,
                     aux_in=bias.to(device) if with_bias else None)
    expect = _expected_grouped(lambda p, slot: x[slot // k], w, seg, N)
    seg_starts, counts, _ = _layout(seg)
    valid = torch.zeros(seg.max_rows, dtype=torch.bool)
    for e in range(E):
        s, c = int(seg_starts[e]), int(counts[e])
        valid[s : s + c] = True
        if with_bias:
            expect[s : s + c] += bias[e].float()
    y_c, act_c = y.float().cpu(), act.float().cpu()
    torch.testing.assert_close(y_c[valid], expect[valid], rtol=RTOL, atol=ATOL)
    torch.testing.assert_close(act_c[valid], F.gelu(expect[valid], approximate="tanh"), rtol=RTOL, atol=ATOL)
    # from the rounded y, like the module applied to y: at most one rounding step of the output type apart
    eps = 2.0**-8 if dtype == torch.bfloat16 else 2.0**-11
    same_input = F.gelu(y.cpu()[valid].float(), approximate="tanh")
    assert float(((act_c[valid] - same_input).abs() / (same_input.abs() + 1e-3)).max()) <= 2 * eps
    assert torch.all(act_c[~valid] == 9.0)  # pad rows are not written


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("n", [8 * 1000, 12345])
def test_gelu_tanh_backward_kernel(device, dtype, n):
    g = torch.Generator().manual_seed(n)
    pre = (2.5 * torch.randn(n, generator=g)).to(dtype)
    d_act = torch.randn(n, generator=g).to(dtype)
    out = torch.empty(n, dtype=dtype, device=device)
    pre_d, d_act_d = pre.to(device), d_act.to(device)
    _C.check(_C.lib().ck_gelu_tanh_bwd(_C.ptr(pre_d), _C.ptr(d_act_d), _C.ptr(out), n, _C.dtype_code(dtype), _C.stream()))
    p64 = pre.double().requires_grad_()
    F.gelu(p64, approximate="tanh").backward(d_act.double())
    torch.testing.assert_close(out.cpu().double(), p64.grad, rtol=RTOL, atol=ATOL)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("epilogue", ["grouped", "scatter"])
@pytest.mark.parametrize("n_out,n_in", [(64, 128), (192, 264), (576, 840), (128, 8)])
def test_grouped_gemm_input_gradient_form(device, dtype, epilogue, n_out, n_in):
    """out = d_y @ w[e] with w [E, n_out, n_in] as the forward stores it (read contraction-strided) equals the same
    product through an explicitly transposed copy, bit for bit (same tiles, same accumulation order), and the fp64 value
    within the 16-bit tolerance."""
    T, k, E = 300, 2, 5
    g, seg = _make_case(device, dtype, T, k, E, 256, seed=7)
    d_y = torch.randn(seg.max_rows, n_out, generator=g).to(dtype)
    w = (0.1 * torch.randn(E, n_out, n_in, generator=g)).to(dtype)
    epi = _C.CK_EPI_GROUPED if epilogue == "grouped" else _C.CK_EPI_SCATTER
    rows = seg.max_rows if epilogue == "grouped" else T * k
    out = torch.zeros(rows, n_in, dtype=dtype, device=device)
    ref = torch.zeros(rows, n_in, dtype=dtype, device=device)
    scattermoe._gemm_dx(d_y.to(device), w.to(device), seg, epi, out)
    scattermoe._gemm(d_y.to(device), 0, w.to(device).transpose(1, 2).contiguous(), seg, epi, ref)
    assert torch.equal(out, ref)
    seg_starts, counts, row_slot = _layout(seg)
    for e in range(E):
        s0, c = int(seg_starts[e]), int(counts[e])
        if c == 0:
            continue
        expect = (d_y[s0 : s0 + c].double() @ w[e].double()).float()
        got = out[s0 : s0 + c] if epilogue == "grouped" else out[torch.from_numpy(row_slot[s0 : s0 + c].astype("int64")).to(device)]
        torch.testing.assert_close(got.float().cpu(), expect, rtol=RTOL, atol=ATOL)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("align", [128, 256])
@pytest.mark.parametrize("K,I", [(200, 72), (128, 256), (64, 136), (96, 440), (192, 440)])
@pytest.mark.parametrize("kind", ["swiglu", "glu"])
def test_grouped_gemm_swiglu_epilogues(device, dtype, align, K, I, gemm_tile, kind):
    """Gated-activation epilogues of the c_fc GEMM: packed SwiGLU (up * silu(gate)) and torch.nn.GLU (up * sigmoid(gate),
    the activation of the reference's MoE test, tests/test_commons.py:85), forward and both backward forms."""
    T, k, E = 300, 2, 5
    glu = kind == "glu"
    act_fn = (lambda t: F.glu(t, dim=-1)) if glu else mo.swiglu_packed_torch
    g, seg = _make_case(device, dtype, T, k, E, align, seed=2)
    x = torch.randn(T, K, generator=g).to(dtype)
    w = (0.1 * torch.randn(E, 2 * I, K, generator=g)).to(dtype)
    pre = torch.zeros(seg.max_rows, 2 * I, dtype=dtype, device=device)
    act = torch.zeros(seg.max_rows, I, dtype=dtype, device=device)
    act_t = torch.full((I, seg.ld_t), 7.0, dtype=dtype, device=device)
    scattermoe._gemm(x.to(device), k, w.to(device), seg, _C.CK_EPI_GLU if glu else _C.CK_EPI_SWIGLU, pre, y_t=act_t, aux=act)
    live = int(seg.seg_starts[E])
    expect_pre = _expected_grouped(lambda p, slot: x[slot // k], w, seg, 2 * I)
    torch.testing.assert_close(pre.float().cpu()[:live], expect_pre[:live], rtol=RTOL, atol=ATOL)
    # the activation is computed from the ROUNDED pre-activation, like the unfused path
    expect_act = act_fn(pre.cpu().float()).to(dtype)
    torch.testing.assert_close(act.cpu()[:live], expect_act[:live], rtol=RTOL, atol=1e-3)
    assert torch.equal(act_t.cpu()[:, :live], act.cpu()[:live].t())

    # backward epilogue: GEMM result is d_act, epilogue applies the SwiGLU backward with the saved pre-activation
    H = K
    d_y = torch.randn(seg.max_rows, H, generator=g).to(dtype)
    w_proj_t = (0.1 * torch.randn(E, I, H, generator=g)).to(dtype)  # [E, I, H]: d_act = d_y @ w_proj
    d_pre = torch.zeros(seg.max_rows, 2 * I, dtype=dtype, device=device)
    d_pre_t = torch.full((2 * I, seg.ld_t), 7.0, dtype=dtype, device=device)
    d_act = _expected_grouped(lambda p, slot: d_y[p], w_proj_t, seg, I).to(dtype)
    pre_c = pre.cpu().float().requires_grad_()
    act_fn(pre_c).backward(d_act.float())
    seg_starts, counts, _ = _layout(seg)
    valid = torch.zeros(seg.max_rows, dtype=torch.bool)
    for e in range(E):
        valid[int(seg_starts[e]) : int(seg_starts[e]) + int(counts[e])] = True
    if not glu:  # the fused backward epilogue exists for SwiGLU only
        scattermoe._gemm(d_y.to(device), 0, w_proj_t.to(device), seg, _C.CK_EPI_SWIGLU_BWD, d_pre, y_t=d_pre_t, aux_in=pre)
        torch.testing.assert_close(d_pre.float().cpu()[valid], pre_c.grad[valid], rtol=2e-2, atol=2e-2)
        assert torch.equal(d_pre_t.cpu()[:, :live], (d_pre.cpu()[:live] * valid[:live, None]).t())

    # the same backward as a plain GEMM followed by the streaming SwiGLU-backward pass (what the layer uses)
    d_act_gpu = torch.zeros(seg.max_rows, I, dtype=dtype, device=device)
    scattermoe._gemm(d_y.to(device), 0, w_proj_t.to(device), seg, _C.CK_EPI_GROUPED, d_act_gpu)
    d_pre2 = torch.zeros(seg.max_rows, 2 * I, dtype=dtype, device=device)
    d_pre2_t = torch.full((2 * I, seg.ld_t), 7.0, dtype=dtype, device=device)
    _C.check(
        _C.lib().ck_swiglu_bwd_grouped(
            pre.data_ptr(), d_act_gpu.data_ptr(), I, seg.seg_starts.data_ptr(), seg.counts.data_ptr(),
            seg.tile_expert.data_ptr(), seg.align, seg.max_rows, d_pre2.data_ptr(), d_pre2_t.data_ptr(), seg.ld_t,
            _C.CK_ACT_GLU if glu else _C.CK_ACT_SWIGLU, _C.dtype_code(dtype), torch.cuda.current_stream().cuda_stream,
        )
    )
    torch.testing.assert_close(d_pre2.float().cpu()[valid], pre_c.grad[valid], rtol=2e-2, atol=2e-2)
    assert torch.equal(d_pre2_t.cpu()[:, :live], (d_pre2.cpu()[:live] * valid[:live, None]).t())
    # without a transposed copy (the layer's call) the whole-row kernel runs: bit-identical rows, pad rows untouched
    d_pre3 = torch.full((seg.max_rows, 2 * I), 5.0, dtype=dtype, device=device)
    _C.check(
        _C.lib().ck_swiglu_bwd_grouped(
            pre.data_ptr(), d_act_gpu.data_ptr(), I, seg.seg_starts.data_ptr(), seg.counts.data_ptr(),
            seg.tile_expert.data_ptr(), seg.align, seg.max_rows, d_pre3.data_ptr(), None, seg.ld_t,
            _C.CK_ACT_GLU if glu else _C.CK_ACT_SWIGLU, _C.dtype_code(dtype), torch.cuda.current_stream().cuda_stream,
        )
    )
    assert torch.equal(d_pre3.cpu()[valid], d_pre2.cpu()[valid])
    assert bool((d_pre3.cpu()[~valid] == 5.0).all())


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("align", [128, 256])
@pytest.mark.parametrize("M,N", [(136, 200), (72, 64), (1024, 1032)])
def test_grouped_gemm_dw(device, dtype, align, M, N, gemm_tile):
    T, k, E = 300, 2, 5
    g, seg = _make_case(device, dtype, T, k, E, align, seed=3)
    a = torch.randn(T * k, M, generator=g).to(dtype)  # (token, slot) order
    b = torch.randn(T, N, generator=g).to(dtype)
    _, a_t = scattermoe._group_rows(a.to(device), None, 1, seg, False, True)
    _, b_t = scattermoe._group_rows(b.to(device), None, k, seg, False, True)
    dw = torch.full((E, M, N), float("nan"), dtype=dtype, device=device)
    scattermoe._gemm_dw(a_t, b_t, seg, dw)
    seg_starts, counts, row_slot = _layout(seg)
    expect = torch.zeros(E, M, N)
    for e in range(E):
        slots = [int(row_slot[p]) for p in range(int(seg_starts[e]), int(seg_starts[e]) + int(counts[e]))]
        if slots:
            expect[e] = a[slots].float().t() @ b[[s // k for s in slots]].float()  # kernels.py:136-222: X^T DY per expert
    torch.testing.assert_close(dw.float().cpu(), expect, rtol=RTOL, atol=0.15)  # sums of ~100 O(1) products
    assert float(dw[3].abs().max()) == 0.0  # empty expert: exact zeros (ops.py:252, kernels.py:181)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("align", [128, 256])
@pytest.mark.parametrize("M,N", [(256, 256), (264, 520), (1024, 1032)])
@pytest.mark.parametrize("T", [900, 40, 100])
def test_grouped_gemm_dw_from_row_major_operands(device, dtype, align, M, N, T):
    """ck_grouped_gemm_dw_rows: X^T DY per expert (kernels.py:136-222) read from the padded-grouped row-major buffers.
    Pad rows are filled with NaN: they must not reach the product. Segments are ragged (counts that are not multiples of
    the 64-row K step, one empty; T = 40: every expert inside a single K step, T = 100: one or two steps)."""
    k, E = 2, 5
    g, seg = _make_case(device, dtype, T, k, E, align, seed=3)
    seg_starts, counts, row_slot = _layout(seg)
    a = torch.full((seg.max_rows, M), float("nan"), dtype=dtype)
    b = torch.full((seg.max_rows, N), float("nan"), dtype=dtype)
    expect = torch.zeros(E, M, N)
    for e in range(E):
        lo, n = int(seg_starts[e]), int(counts[e])
        a[lo : lo + n] = torch.randn(n, M, generator=g).to(dtype)
        b[lo : lo + n] = torch.randn(n, N, generator=g).to(dtype)
        if n:
            expect[e] = a[lo : lo + n].float().t() @ b[lo : lo + n].float()
    assert int(counts.min()) == 0 and any(int(c) % 64 for c in counts)
    dw = torch.full((E, M, N), float("nan"), dtype=dtype, device=device)
    scattermoe._gemm_dw_rows(a.to(device), b.to(device), seg, dw)
    torch.testing.assert_close(dw.float().cpu(), expect, rtol=RTOL, atol=0.3)  # sums of up to ~700 O(1) products
    assert float(dw[3].abs().max()) == 0.0  # empty expert: exact zeros (ops.py:252, kernels.py:181)


def test_grouped_gemm_grouped_input_beyond_4_gib(device):
    """A padded-grouped input of 4.9 GB (600,000 rows x 4,096 bf16): rows are addressed from each tile's first row, so the
    32-bit offsets inside the kernels never see the size of the whole operand. Checked on the last rows of the last expert
    (byte offsets past 2^32) and on the first rows, for the forward form and the input-gradient form, against torch's
    GEMM on the same device."""
    torch.manual_seed(5)
    R, E, K, N = 600_000, 2, 4096, 256
    ids = (torch.arange(R, dtype=torch.int32) >= 250_000).to(torch.int32)  # expert 0: 250,000 rows, expert 1: 350,000
    seg = cute_kernels.sort_by_expert(ids.to(device), E, 256)
    assert seg.max_rows * K * 2 > 2**32
    a = torch.randn(seg.max_rows, K, device=device, dtype=torch.bfloat16)
    w = (0.05 * torch.randn(E, N, K, device=device)).to(torch.bfloat16)
    y = torch.zeros(seg.max_rows, N, dtype=torch.bfloat16, device=device)
    scattermoe._gemm(a, 0, w, seg, _C.CK_EPI_GROUPED, y)
    seg_starts, counts, _ = _layout(seg)
    last = int(seg_starts[1]) + int(counts[1])
    for lo, hi, e in ((0, 512, 0), (last - 1000, last, 1)):
        want = a[lo:hi].float() @ w[e].float().t()
        torch.testing.assert_close(y[lo:hi].float(), want, rtol=RTOL, atol=2e-2)
    # input-gradient form: x = a @ w_nn[e] with w_nn [E, K, N2] read as stored
    w_nn = (0.05 * torch.randn(E, K, 512, device=device)).to(torch.bfloat16)
    y2 = torch.zeros(seg.max_rows, 512, dtype=torch.bfloat16, device=device)
    scattermoe._gemm_dx(a, w_nn, seg, _C.CK_EPI_GROUPED, y2)
    want = a[last - 1000 : last].float() @ w_nn[1].float()
    torch.testing.assert_close(y2[last - 1000 : last].float(), want, rtol=RTOL, atol=2e-2)


# ---------------------------------------------------------------------------------------------------------------
# whole layer
# ---------------------------------------------------------------------------------------------------------------
class _OracleWithSelection(mo.MoEOracle):
    """The oracle layer with the expert selection supplied from outside. A one-ulp difference between two router GEMMs
    can flip a near-tie and swap whole experts; selection itself is pinned bit-exactly in test_gpu_routing.py, so here
    both sides route identically and everything downstream (gates included) is compared numerically."""

    forced_selection = None

    def _compute_routing_weights(self, hidden_states):
        router_logits = self.gate(hidden_states)
        sel = self.forced_selection
        vals = router_logits.gather(-1, sel)
        weights = F.softmax(vals.float(), dim=-1).type_as(hidden_states)
        if weights.requires_grad:
            weights.retain_grad()
        self.last_router_weights = weights
        return router_logits, weights, sel


def _close_via_truth(ours, oracle, truth, what, rtol=RTOL, atol=ATOL, rms_margin=2e-3):
    """Per element: within atol * s + rtol * |x| of the oracle, or no further from the fp32 truth than the oracle is plus
    that margin, where s is the RMS of the tensor (the absolute tolerance is stated in units of the tensor's typical
    magnitude, so that it cannot exceed the signal it checks). Over the whole tensor: our RMS distance to the truth is at
    most 1.1 x the oracle's -- an all-zero, mis-scaled or permuted result fails this whatever the tolerances."""
    ours, oracle, truth = ours.detach().float().cpu(), oracle.detach().float().cpu(), truth.detach().float().cpu()
    nonzero = int((truth != 0).sum())  # weight gradients of experts that received no token are exact zeros: leave them out of the scale
    if nonzero == 0:  # e.g. gate.weight.grad with top-1 routing (a softmax over one logit is constant)
        assert float(ours.abs().max()) <= 1e-3 and float(oracle.abs().max()) <= 1e-3, f"{what}: should vanish"
        return
    scale = float((truth.square().sum() / nonzero).sqrt())
    direct = (ours - oracle).abs() <= atol * scale + rtol * oracle.abs()
    via = (ours - truth).abs() <= (oracle - truth).abs() + atol * scale + rtol * truth.abs()
    bad = ~(direct | via)
    worst_ours, worst_oracle = float((ours - truth).abs().max()), float((oracle - truth).abs().max())
    # one element per million may miss the per-element bound (a gate-weighted sum of rounded rows that cancel), but none
    # may be further from the truth than 1.25 x the oracle's own worst element
    assert int(bad.sum()) <= bad.numel() // 1_000_000 and worst_ours <= 1.25 * worst_oracle + atol * scale, (
        f"{what}: {int(bad.sum())}/{bad.numel()} elements off; worst |ours-oracle|={float((ours - oracle).abs().max()):.4g}, "
        f"|ours-truth|={worst_ours:.4g}, |oracle-truth|={worst_oracle:.4g}, rms={scale:.4g}"
    )
    err_ours = float(((ours - truth).square().sum() / nonzero).sqrt())
    err_oracle = float(((oracle - truth).square().sum() / nonzero).sqrt())
    assert err_ours <= 1.1 * err_oracle + rms_margin * scale, f"{what}: RMS error {err_ours:.4g} against the oracle's {err_oracle:.4g} (rms {scale:.4g})"


def _acts(name):
    if name == "swiglu":
        return cute_kernels.swiglu_packed_cute, mo.swiglu_packed_torch, True
    if name == "glu":  # the reference test's own activations (tests/test_commons.py:85-86)
        return nn.GLU(), nn.GLU(), True
    return nn.GELU(approximate="tanh"), nn.GELU(approximate="tanh"), False


def _run_layer_case(device, dtype, T, E, k, H, I, act_name, x_shape=None, seed=42, add_bias=False, moe_cls=None,
                    x_grad_atol=2e-2):
    # fp32 layers (fp32 MFMA, fp32 accumulation) are held to 1e-4 instead of 1e-2: two orders tighter than the 16-bit bars
    tol = 1e-2 if dtype == torch.float32 else 1.0
    torch.manual_seed(seed)
    act_gpu, act_cpu, is_glu = _acts(act_name)
    # weights ~ N(0, 1 / fan_in-ish): pre-activations, outputs and gradients are O(1), so the tolerances below (stated
    # relative to each tensor's RMS) check real digits
    std = 1.0 / (H ** 0.5)
    moe = (moe_cls or cute_kernels.MoE)(E, k, H, I, act_gpu, is_glu, add_bias, std).to(dtype)
    if add_bias:  # the constructor zeroes biases (torch_implementation.py:56-60); give them values
        with torch.no_grad():
            moe.c_fc.bias.normal_(0, 0.1)
            moe.c_proj.bias.normal_(0, 0.1)
    oracle = _OracleWithSelection(E, k, H, I, act_cpu, is_glu, add_bias, std).to(dtype)
    oracle.load_state_dict(moe.state_dict())  # same state_dict keys as the reference (scattermoe_test.py:83-94)
    truth = _OracleWithSelection(E, k, H, I, act_cpu, is_glu, add_bias, std).float()
    truth.load_state_dict({n: v.float() for n, v in moe.state_dict().items()})
    moe = moe.to(device)

    x = torch.randn(x_shape or (T, H)).to(dtype)
    r = torch.randn(x.shape).to(dtype)  # random cotangent (the reference uses ones: y.sum())
    xg = x.clone().to(device).requires_grad_()
    xo = x.clone().requires_grad_()
    xt = x.clone().float().requires_grad_()

    captured = {}
    orig = moe._compute_routing_weights

    def spy(hs):
        out = orig(hs)
        captured["sel"] = out[2].detach().cpu()
        captured["weights"] = out[1].detach().cpu()
        return out

    moe._compute_routing_weights = spy
    y, logits = moe(xg)
    oracle.forced_selection = truth.forced_selection = captured["sel"]
    yo, logits_o = oracle(xo)
    yt, _ = truth(xt)
    assert y.shape == x.shape and logits.shape == (x.numel() // H, E) and y.dtype == dtype

    torch.testing.assert_close(logits.float().cpu(), logits_o.float(), rtol=RTOL * tol, atol=ATOL * tol)
    _close_via_truth(y, yo.detach(), yt.detach(), "output", rtol=RTOL * tol, atol=ATOL * tol, rms_margin=2e-3 * tol)

    (y * r.to(device)).sum().backward()
    (yo * r).sum().backward()
    (yt * r.float()).sum().backward()
    _close_via_truth(xg.grad, xo.grad, xt.grad, "x.grad", rtol=RTOL * tol, atol=x_grad_atol * tol, rms_margin=2e-3 * tol)
    for name in ["c_fc", "c_proj"]:
        _close_via_truth(
            getattr(moe, name).weight.grad, getattr(oracle, name).weight.grad, getattr(truth, name).weight.grad,
            f"{name}.weight.grad", rtol=RTOL * tol, atol=3e-2 * tol, rms_margin=2e-3 * tol,
        )
    if add_bias:
        for name in ["c_fc", "c_proj"]:
            _close_via_truth(
                getattr(moe, name).bias.grad, getattr(oracle, name).bias.grad, getattr(truth, name).bias.grad,
                f"{name}.bias.grad", rtol=RTOL * tol, atol=3e-2 * tol, rms_margin=2e-3 * tol,
            )
    # d_gates stays in fp32 between the expert block's backward and the router's (the reference rounds it to the
    # activation dtype, ops.py:214, and so does the oracle): same tolerance as the other weight gradients
    _close_via_truth(moe.gate.weight.grad, oracle.gate.weight.grad, truth.gate.weight.grad, "gate.weight.grad",
                     rtol=RTOL * tol, atol=3e-2 * tol, rms_margin=2e-3 * tol)
    return moe, oracle


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("act", ["swiglu", "glu", "gelu"])
@pytest.mark.parametrize("T,E,k,H,I", [(257, 8, 2, 128, 256), (33, 4, 4, 64, 72), (700, 64, 8, 128, 136), (1, 6, 2, 256, 64)])
def test_moe_layer_forward_backward(device, dtype, act, T, E, k, H, I):
    _run_layer_case(device, dtype, T, E, k, H, I, act)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])  # the dtypes of tests/test_commons.py:26-27
@pytest.mark.parametrize(
    "E,k,H,I",
    # every combination of scattermoe_test.py:17-38 that its own skip (k > E) leaves: E in {2, 4, 6, 8} x k in {2, 4} at
    # H = 2048, I = 8192, and (128, 8, 576, 256)
    [(2, 2, 2048, 8192), (4, 2, 2048, 8192), (4, 4, 2048, 8192), (6, 2, 2048, 8192), (6, 4, 2048, 8192), (8, 2, 2048, 8192),
     (8, 4, 2048, 8192), (128, 8, 576, 256)],
)
@pytest.mark.parametrize("act", ["glu", "gelu"])
def test_moe_layer_reference_test_shapes_single_token(device, dtype, E, k, H, I, act):
    # scattermoe_test.py:17-127: x = randn(hidden_size), one token, 1-D input
    _run_layer_case(device, dtype, 1, E, k, H, I, act, x_shape=(H,))


def test_moe_layer_3d_input_top1_and_large_tiles(device):
    _run_layer_case(device, torch.bfloat16, 0, 4, 1, 64, 72, "swiglu", x_shape=(3, 50, 64))
    # enough rows per expert for the 256-row tile path (choose_align), Zipf-free but ragged
    _run_layer_case(device, torch.bfloat16, 9000, 4, 2, 128, 136, "swiglu")


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("act", ["swiglu", "glu", "gelu"])
@pytest.mark.parametrize("T,E,k,H,I", [(257, 8, 2, 128, 256), (33, 4, 4, 64, 72), (700, 64, 8, 128, 136), (3000, 4, 2, 128, 256)])
def test_moe_layer_with_expert_biases(device, dtype, act, T, E, k, H, I):
    # add_bias=True: the reference's torch path applies one bias row per expert (torch_implementation.py:20-22,42); its
    # Triton path drops them, so the reference's own test only runs add_bias=False (scattermoe_test.py:62-77).
    # The last shape has 256-row tiles and contraction lengths that are multiples of 64: there the bias is an operand of
    # the GEMM epilogues; the others add it with its own kernel.
    _run_layer_case(device, dtype, T, E, k, H, I, act, add_bias=True)


def test_moe_layer_rejects_unsupported_dtypes(device):
    moe = cute_kernels.MoE(4, 2, 64, 72, cute_kernels.swiglu_packed_cute, True, False, 0.02).double().to(device)
    with pytest.raises((NotImplementedError, ValueError, AssertionError)):
        moe(torch.randn(5, 64, device=device, dtype=torch.float64))


@pytest.mark.parametrize("w_is_kn", [False, True])
@pytest.mark.parametrize("scatter", [False, True])
@pytest.mark.parametrize("align,K,N", [(128, 200, 136), (256, 64, 128), (128, 24, 8), (256, 100, 332)])
def test_grouped_gemm_f32(device, align, K, N, scatter, w_is_kn):
    """ck_grouped_gemm_f32 against fp64 per-expert products: fp32 MFMA products with fp32 accumulation, rtol = atol = 1e-5
    on O(1) outputs (bias included); gathered input, both weight layouts, both output orders."""
    T, k, E = 300, 2, 5
    g, seg = _make_case(device, torch.float32, T, k, E, align, seed=5)
    x = torch.randn(T, K, generator=g)
    w = torch.randn(E, N, K, generator=g) * K**-0.5
    bias = torch.randn(E, N, generator=g)
    w_dev = (w.transpose(1, 2).contiguous() if w_is_kn else w).to(device)
    rows = T * k if scatter else seg.max_rows
    y = torch.full((rows, N), 7.0, device=device)
    scattermoe._gemm_f32(x.to(device), k, w_dev, w_is_kn, N, K, seg, scatter, y, bias.to(device))
    seg_starts, counts, row_slot = _layout(seg)
    y_c = y.cpu()
    written = torch.zeros(rows, dtype=torch.bool)
    for e in range(E):
        s, c = int(seg_starts[e]), int(counts[e])
        for p in range(s, s + c):
            slot = int(row_slot[p])
            want = (x[slot // k].double() @ w[e].double().t() + bias[e].double()).float()
            out_row = slot if scatter else p
            written[out_row] = True
            torch.testing.assert_close(y_c[out_row], want, rtol=1e-5, atol=1e-5)
    assert torch.all(y_c[~written] == 7.0)  # pad rows are not written
    assert not scatter or bool(written.all())


@pytest.mark.parametrize("align,M,N", [(128, 136, 200), (256, 64, 64), (128, 8, 332)])
def test_grouped_gemm_dw_f32(device, align, M, N):
    T, k, E = 300, 2, 5
    g, seg = _make_case(device, torch.float32, T, k, E, align, seed=6)
    a = torch.randn(seg.max_rows, M, generator=g)
    b = torch.randn(seg.max_rows, N, generator=g)
    dw = torch.full((E, M, N), 3.0, device=device)
    scattermoe._gemm_dw_rows(a.to(device), b.to(device), seg, dw)
    seg_starts, counts, _ = _layout(seg)
    for e in range(E):
        s, c = int(seg_starts[e]), int(counts[e])
        want = (a[s : s + c].double().t() @ b[s : s + c].double()).float()  # exact zeros for an expert without rows
        torch.testing.assert_close(dw[e].cpu(), want, rtol=1e-5, atol=1e-5 * max(1.0, c**0.5))


def test_moe_fused_path_equals_unfused_path_at_mixtral_row_shape(device):
    """Size-independent property at the baseline's hidden sizes (T reduced to keep the unfused reference small): the
    fused SwiGLU expert block and the three-kernel unfused path (GEMM -> swiglu_packed_cute -> GEMM) agree, forward and
    input gradient, and the output is invariant under a permutation of the tokens."""
    torch.manual_seed(0)
    E, k, H, I, T = 8, 2, 4096, 14336, 2048
    dtype = torch.bfloat16
    moe = cute_kernels.MoE(E, k, H, I, cute_kernels.swiglu_packed_cute, True, False, 0.02).to(dtype).to(device)
    x = torch.randn(T, H, device=device, dtype=dtype)
    xa = x.clone().requires_grad_()
    ya, _ = moe(xa)
    ya.sum().backward()
    moe.act = lambda v: cute_kernels.swiglu_packed_cute(v)  # a different callable: takes the generic path
    xb = x.clone().requires_grad_()
    yb, _ = moe(xb)
    yb.sum().backward()
    torch.testing.assert_close(ya, yb, rtol=RTOL, atol=ATOL)
    torch.testing.assert_close(xa.grad, xb.grad, rtol=RTOL, atol=2e-2)
    moe.act = cute_kernels.swiglu_packed_cute
    perm = torch.randperm(T, device=device)
    with torch.no_grad():
        yp, _ = moe(x[perm])
    torch.testing.assert_close(yp, ya.detach()[perm], rtol=RTOL, atol=ATOL)


def _close_via_truth_on_device(ours, oracle, truth, what, rtol=RTOL, atol=ATOL):
    """Per element: within atol * s + rtol * |x| of the bf16 oracle, or no further from the fp32 truth than the oracle is
    plus that margin; s = max(1, RMS of the tensor): at these sizes outputs and gradients are sums of thousands of O(1)
    terms, and the absolute tolerance is stated in units of their typical magnitude. At most one element in a million may
    miss that bound (an output element is a gate-weighted sum of per-expert rows that are themselves rounded to bf16:
    where large rows cancel, the rounding of the parts exceeds any tolerance tied to the sum), and no element may be
    further from the truth than 1.25 x the oracle's own worst element. Over the whole tensor: our RMS distance to the
    truth is at most 1.1 x the oracle's."""
    ours, oracle, truth = ours.detach().float(), oracle.detach().float(), truth.detach().float()
    scale = max(1.0, float(truth.square().mean().sqrt()))
    direct = (ours - oracle).abs() <= atol * scale + rtol * oracle.abs()
    via = (ours - truth).abs() <= (oracle - truth).abs() + atol * scale + rtol * truth.abs()
    bad = ~(direct | via)
    err_ours = float((ours - truth).square().mean().sqrt())
    err_oracle = float((oracle - truth).square().mean().sqrt())
    worst_ours, worst_oracle = float((ours - truth).abs().max()), float((oracle - truth).abs().max())
    assert int(bad.sum()) <= bad.numel() // 1_000_000 and worst_ours <= 1.25 * worst_oracle + atol * scale, (
        f"{what}: {int(bad.sum())}/{bad.numel()} elements off; worst |ours-oracle|={float((ours - oracle).abs().max()):.4g}, "
        f"|ours-truth|={worst_ours:.4g}, |oracle-truth|={worst_oracle:.4g}"
    )
    assert err_ours <= 1.1 * err_oracle + 1e-3 * scale, f"{what}: RMS error {err_ours:.4g} against the oracle's {err_oracle:.4g}"


@pytest.mark.parametrize(
    "name,T,E,k,H,I,skew,norm",
    [("C3", 16384, 8, 2, 4096, 14336, 0.5, False), ("C3-gates-rewrapped", 16384, 8, 2, 4096, 14336, 0.5, False),
     ("C4", 8192, 64, 8, 2048, 1408, 0.0, True), ("C4-fused-prologue", 8192, 64, 8, 2048, 1408, 0.0, "fused")],
)
def test_moe_layer_at_full_baseline_shapes(device, monkeypatch, name, T, E, k, H, I, skew, norm):
    """The benchmark's own workloads, forward and every gradient, against the oracle layer evaluated by torch's library
    routines on the same device (bf16, and fp32 as the truth that arbitrates rounding): same tolerances as the small
    cases. `skew` > 0 adds the benchmark's rank-dependent router bias so that expert loads are ragged (Zipf-like);
    `norm` puts the RMSNorm prologue (eps 1e-6, weight ~ N(1, 0.02)) in front of the layer as bench.py does for C4:
    rmsnorm_cute on our side, F.rms_norm in the oracle, gradients taken through it. norm == "fused" is the route the
    benchmark's C4 step takes: MoE.forward_with_norm, one kernel for the normalised rows and the router logits, with its
    own backward; the oracle side is the same composition, routed by the selection the layer made on its own logits (that
    selection is compared bit-exactly with the oracle's top-k rule applied to those logits).
    "C3-gates-rewrapped": something between the router and the experts hands on a new gates tensor (a clone here; autocast,
    a user hook or .to() do the same), so the fp32 d_gates the expert block leaves for the router's backward is not found
    and gate.weight.grad is computed from the 16-bit gradient autograd delivers, as in the reference (ops.py:214): held to
    the same bounds."""
    torch.manual_seed(7)
    dtype = torch.bfloat16
    moe = cute_kernels.MoE(E, k, H, I, cute_kernels.swiglu_packed_cute, True, False, 0.02).to(dtype)
    oracle = _OracleWithSelection(E, k, H, I, mo.swiglu_packed_torch, True, False, 0.02).to(dtype)
    oracle.load_state_dict(moe.state_dict())
    truth = _OracleWithSelection(E, k, H, I, mo.swiglu_packed_torch, True, False, 0.02).float()
    truth.load_state_dict({n: v.float() for n, v in moe.state_dict().items()})
    moe, oracle, truth = moe.to(device), oracle.to(device), truth.to(device)
    bias = (-skew * torch.log(torch.arange(1, E + 1, dtype=torch.float32))).to(device)
    for layer in (moe, oracle, truth):
        layer.gate.register_forward_hook(lambda mod, inp, out: out + bias.to(out.dtype))

    x = torch.randn(T, H, generator=torch.Generator().manual_seed(1)).to(dtype).to(device)
    r = torch.randn(T, H, generator=torch.Generator().manual_seed(2)).to(dtype).to(device)
    xg, xo, xt = x.clone().requires_grad_(), x.clone().requires_grad_(), x.clone().float().requires_grad_()
    hg, ho, ht = xg, xo, xt  # what the layer sees
    if norm:
        w_n = (1 + 0.02 * torch.randn(H, generator=torch.Generator().manual_seed(3))).to(dtype).to(device)
        wg, wo, wt = w_n.clone().requires_grad_(), w_n.clone().requires_grad_(), w_n.clone().float().requires_grad_()
        hg = cute_kernels.rmsnorm_cute(xg, wg, 1e-6)
        ho = mo.rmsnorm_torch(xo, wo, 1e-6)
        ht = mo.rmsnorm_torch(xt, wt, 1e-6)

    captured = {}
    if norm == "fused":
        from cute_kernels.modules import moe as moe_module

        real_route = moe_module.route_topk_softmax

        def route_spy(router_logits, top_k):
            out = real_route(router_logits, top_k)
            captured["sel"] = out[1].detach()
            return out

        monkeypatch.setattr(moe_module, "route_topk_softmax", route_spy)
        y, logits = moe.forward_with_norm(xg, wg, 1e-6)
        # the selection is the oracle's rule (k largest, lowest index first among equals) applied to the kernel's own logits
        want = torch.sort(logits.detach().float(), dim=-1, descending=True, stable=True).indices[:, :k]
        assert torch.equal(captured["sel"], want)
    else:
        orig = moe._compute_routing_weights

        def spy(hs):
            out = orig(hs)
            captured["sel"] = out[2].detach()
            if name == "C3-gates-rewrapped":
                rewrapped = out[1].clone()
                assert scattermoe._gate_slot(out[1]) is not None and scattermoe._gate_slot(rewrapped) is None
                return out[0], rewrapped, out[2]
            return out

        moe._compute_routing_weights = spy
        y, logits = moe(hg)
    oracle.forced_selection = truth.forced_selection = captured["sel"]
    load = torch.bincount(captured["sel"].flatten(), minlength=E).float() / (T * k)
    if skew > 0:
        assert float(load.max()) > 2.5 * float(load.min())  # ragged segments really are exercised
    yo, logits_o = oracle(ho)
    yt, _ = truth(ht)
    torch.testing.assert_close(logits.float(), logits_o.float(), rtol=RTOL, atol=ATOL)
    _close_via_truth_on_device(y, yo.detach(), yt.detach(), f"{name} output")

    (y * r).sum().backward()
    (yo * r).sum().backward()
    (yt * r.float()).sum().backward()
    _close_via_truth_on_device(xg.grad, xo.grad, xt.grad, f"{name} x.grad", atol=2e-2)
    if norm:
        _close_via_truth_on_device(wg.grad, wo.grad, wt.grad, f"{name} rmsnorm weight.grad", atol=3e-2)
    for pname in ["c_fc", "c_proj"]:
        _close_via_truth_on_device(
            getattr(moe, pname).weight.grad, getattr(oracle, pname).weight.grad, getattr(truth, pname).weight.grad,
            f"{name} {pname}.weight.grad", atol=3e-2,
        )
    _close_via_truth_on_device(
        moe.gate.weight.grad, oracle.gate.weight.grad, truth.gate.weight.grad, f"{name} gate.weight.grad", atol=3e-2
    )


@pytest.mark.parametrize("act,kind", [("swiglu", _C.CK_ACT_SWIGLU), ("glu", _C.CK_ACT_GLU), ("gelu", None), ("silu", None)])
def test_known_activations_run_in_the_c_fc_epilogue(device, monkeypatch, act, kind):
    """Packed SwiGLU and torch.nn.GLU run inside the c_fc epilogue (swiglu_experts with the matching act_kind), and so does
    nn.GELU("tanh") (experts_up with gelu_tanh=True); any other callable goes GEMM -> callable -> GEMM. Results of all
    routes are covered by the layer parity tests above."""
    from cute_kernels.modules import moe as moe_module

    act_gpu, is_glu = (nn.SiLU(), False) if act == "silu" else (_acts(act)[0], _acts(act)[2])
    layer = cute_kernels.MoE(4, 2, 128, 256, act_gpu, is_glu, False, 0.02).to(torch.bfloat16).to(device)
    seen, seen_up = [], []
    real, real_up = moe_module.swiglu_experts, moe_module.experts_up
    monkeypatch.setattr(moe_module, "swiglu_experts", lambda *a: (seen.append(a[5]), real(*a))[1])
    monkeypatch.setattr(moe_module, "experts_up", lambda *a, **kw: (seen_up.append(kw.get("gelu_tanh", False)), real_up(*a, **kw))[1])
    layer(torch.randn(300, 128, device=device, dtype=torch.bfloat16))
    assert seen == ([kind] if kind is not None else [])
    assert seen_up == ({"gelu": [True], "silu": [False]}.get(act, []))


def test_bias_in_the_gemm_epilogue_equals_the_separate_bias_kernel(device, monkeypatch):
    """Same layer, same input, biases on: the epilogue form (one rounding of accumulator + bias) against the GEMM followed
    by ck_add_expert_bias (two roundings): equal within one bf16 rounding step of the outputs, forward and gradients."""
    torch.manual_seed(1)
    layer = cute_kernels.MoE(4, 2, 128, 256, nn.GELU(approximate="tanh"), False, True, 0.02).to(torch.bfloat16).to(device)
    with torch.no_grad():
        layer.c_fc.bias.normal_(0, 0.2)
        layer.c_proj.bias.normal_(0, 0.2)
    x = torch.randn(3000, 128, device=device, dtype=torch.bfloat16)
    results = []
    for fused in (True, False):
        monkeypatch.setattr(scattermoe.options, "bias_fused", fused)
        for p in layer.parameters():
            p.grad = None
        xi = x.clone().requires_grad_()
        y, _ = layer(xi)
        y.float().square().sum().backward()
        results.append((y.detach(), xi.grad, layer.c_fc.bias.grad.clone(), layer.c_proj.bias.grad.clone()))
    for a, b in zip(*results):
        torch.testing.assert_close(a.float(), b.float(), rtol=2e-2, atol=2e-2 * max(1.0, float(b.float().abs().max()) / 8))
    assert not torch.equal(results[0][0], results[1][0])  # the two forms really differ in rounding: both paths ran
