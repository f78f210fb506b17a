"""MoE expert path: routing, token->expert sort, scattered grouped GEMMs, gated combine -- forward and backward.

Semantics follow cute_kernels/kernels/scattermoe/torch_implementation.py:63-201 (reference oracle) and the autograd
conventions of cute_kernels/kernels/scattermoe/triton_implementation/ops.py:143-292. The data layout does not: rows
are kept in a padded grouped order where every expert's segment starts at a multiple of the GEMM tile height, and the
backward GEMMs consume transposed copies that the producing kernels write as they go, so that every matrix product is
contraction-contiguous on both operands.
"""

from __future__ import annotations

import ctypes
from dataclasses import dataclass

import torch

from . import _C
from .utils import is_tracing

_ops = None  # cute_kernels.compile_ops, set by the package once it is imported (used only while torch.compile traces)


@dataclass
class Options:
    """Switches between forms that compute the same result, for tests and measurements (bench.py sets them from its
    command line). The defaults are what the library runs; nothing reads the environment."""

    gemm_split: bool = True  # the last, partial round of GEMM tiles splits its contraction over the idle CUs
    bias_fused: bool = True  # expert biases join the GEMM's fp32 accumulators (False: their own kernel after the GEMM)
    gemm_nn: bool = True  # input-gradient GEMMs read the weight as stored (False: through a transposed copy)
    dw_rows: bool = True  # weight-gradient GEMMs read row-major operands (False: transposed copies)


options = Options()


# ---------------------------------------------------------------------------------------------------------------
# routing
# ---------------------------------------------------------------------------------------------------------------
class _GateGradSlot:
    """Side channel between the expert block's backward and the router's backward. Autograd hands a 16-bit gates tensor
    a 16-bit gradient; the softmax backward then subtracts nearly equal rounded numbers and gate.weight.grad loses
    digits. The expert block leaves its unrounded fp32 d_gates here, and the router's backward uses it when the gradient
    it receives is exactly that tensor rounded (i.e. nothing else contributed to the gates' gradient)."""

    __slots__ = ("d_gates_f32",)

    def __init__(self):
        self.d_gates_f32 = None


def _gate_slot(gates: torch.Tensor):
    return getattr(gates, "_ck_gate_slot", None)


class _RouteTopKSoftmax(torch.autograd.Function):
    """logits [T, E] -> gates [T, k] (softmax over the k largest logits, in logits.dtype), selected [T, k] int64."""

    @staticmethod
    def forward(ctx, logits: torch.Tensor, k: int, long_indices: bool = True, slot: _GateGradSlot | None = None):
        _C.require_gpu(logits)
        logits = logits.contiguous()
        T, E = logits.shape
        selected = torch.empty(T, k, dtype=torch.int32, device=logits.device)
        gates = torch.empty(T, k, dtype=torch.float32, device=logits.device)
        lib = _C.lib()
        with torch.cuda.device(logits.device):
            _C.check(
                lib.ck_route_topk_softmax(
                    _C.ptr(logits), _C.dtype_code(logits.dtype), T, E, k, _C.ptr(selected), _C.ptr(gates), None, _C.stream()
                )
            )
        ctx.save_for_backward(gates, selected)
        ctx.E = E
        ctx.dtype = logits.dtype
        ctx.slot = slot
        selected_out = selected.long() if long_indices else selected
        ctx.mark_non_differentiable(selected_out)
        return gates.to(logits.dtype), selected_out

    @staticmethod
    def backward(ctx, d_gates: torch.Tensor, _d_selected):
        gates, selected = ctx.saved_tensors
        T, k = gates.shape
        exact = ctx.slot.d_gates_f32 if ctx.slot is not None else None
        d_logits = torch.empty(T, ctx.E, dtype=ctx.dtype, device=gates.device)
        lib = _C.lib()
        if exact is not None and exact.shape == d_gates.shape and d_gates.dtype == ctx.dtype != torch.float32:
            # the unrounded gradient wherever what arrived is that gradient rounded (decided per element inside the
            # kernel: no host sync, no extra launches)
            ctx.slot.d_gates_f32 = None
            d_gates = d_gates.contiguous()
            with torch.cuda.device(gates.device):
                _C.check(
                    lib.ck_route_topk_softmax_bwd_exact(
                        _C.ptr(gates), _C.ptr(exact), _C.ptr(d_gates), _C.ptr(selected), T, ctx.E, k, _C.ptr(d_logits),
                        _C.dtype_code(ctx.dtype), _C.stream(),
                    )
                )
            return d_logits, None, None, None
        d_gates = d_gates.float().contiguous()
        with torch.cuda.device(gates.device):
            _C.check(
                lib.ck_route_topk_softmax_bwd(
                    _C.ptr(gates), _C.ptr(d_gates), _C.ptr(selected), T, ctx.E, k, _C.ptr(d_logits),
                    _C.dtype_code(ctx.dtype), _C.stream(),
                )
            )
        return d_logits, None, None, None


def route_topk_softmax(logits: torch.Tensor, k: int, long_indices: bool = True) -> tuple[torch.Tensor, torch.Tensor]:
    """Top-k over the logits and softmax over the k selected logits in fp32, cast back to logits.dtype
    (torch_implementation.py:122-135). Equal logits: the lowest expert index wins. The indices come back as int64 like
    torch.topk's; long_indices=False keeps the kernel's int32 (what the sort consumes fastest)."""
    if is_tracing():
        gates, selected = _ops.route_topk_softmax(logits, k)
        return gates.to(logits.dtype), (selected.long() if long_indices else selected)
    slot = _GateGradSlot()
    gates, selected = _RouteTopKSoftmax.apply(logits, k, long_indices, slot)
    gates._ck_gate_slot = slot  # found again by the expert block that consumes these gates (see _GateGradSlot)
    return gates, selected


@torch.no_grad()
def route_topk_softmax_raw(logits: torch.Tensor, k: int) -> tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """(selected int32 [T, k], gates fp32 [T, k], top-k values [T, k] in logits.dtype), no autograd."""
    _C.require_gpu(logits)
    logits = logits.contiguous()
    T, E = logits.shape
    selected = torch.empty(T, k, dtype=torch.int32, device=logits.device)
    gates = torch.empty(T, k, dtype=torch.float32, device=logits.device)
    values = torch.empty(T, k, dtype=logits.dtype, device=logits.device)
    lib = _C.lib()
    with torch.cuda.device(logits.device):
        _C.check(
            lib.ck_route_topk_softmax(
                _C.ptr(logits), _C.dtype_code(logits.dtype), T, E, k, _C.ptr(selected), _C.ptr(gates), _C.ptr(values),
                _C.stream(),
            )
        )
    return selected, gates, values


# ---------------------------------------------------------------------------------------------------------------
# sort + segments
# ---------------------------------------------------------------------------------------------------------------
@dataclass
class ExpertSegments:
    """Result of the stable sort by expert, in the reference's vocabulary plus the padded grouped layout."""

    sorted_expert_idxs: torch.Tensor  # int32 [R]
    sorted_scattered_idxs: torch.Tensor  # int32 [R]
    counts: torch.Tensor  # uint32 [E]
    ends: torch.Tensor  # uint32 [E]  inclusive prefix sums (the reference's expert_offsets)
    starts: torch.Tensor  # uint32 [E]  exclusive prefix sums
    seg_starts: torch.Tensor  # int32 [E + 1]
    row_slot: torch.Tensor  # int32 [max_rows]
    tile_expert: torch.Tensor  # int32 [max_rows / align]
    max_rows: int
    num_experts: int
    align: int
    # int32 [max_rows]: the sorted position a padded row stands for, i.e. its row in an UNPADDED grouped tensor [R, *]
    # (the reference's grouped_in / grouped_out layout). Only segments_from_sorted fills it.
    row_pos: torch.Tensor | None = None

    def c_struct(self, rows_in: torch.Tensor | None = None, rows_out: torch.Tensor | None = None) -> _C.ck_segments:
        """rows_in: table a gathered input is read through (default row_slot); rows_out: table the scatter epilogue writes
        through (default: the same as rows_in)."""
        rows_in = self.row_slot if rows_in is None else rows_in
        return _C.ck_segments(
            self.seg_starts.data_ptr(),
            self.counts.data_ptr(),
            self.tile_expert.data_ptr(),
            rows_in.data_ptr(),
            self.max_rows,
            self.num_experts,
            self.align,
            None if rows_out is None else rows_out.data_ptr(),
        )

    @property
    def ld_t(self) -> int:
        """Leading dimension of transposed padded-grouped operands."""
        return self.max_rows


def choose_align(num_rows: int, num_experts: int) -> int:
    """Tile height of the padded layout: 256-row tiles once experts average at least 512 rows (measured at the
    fine-grained shape, 1024 rows per expert: 256-row tiles run the forward GEMMs 30 % faster than 128-row ones despite
    the extra padding), else 128."""
    return 256 if num_rows >= 512 * num_experts else 128


@torch.no_grad()
def sort_by_expert(
    expert_ids: torch.Tensor, num_experts: int, align: int | None = None, validate: bool = False
) -> ExpertSegments:
    """Stable sort of the flat (token, slot) expert ids, with counts / offsets and the tile-aligned segment tables.

    Contract: every id lies in [0, num_experts) -- what a top-k over num_experts logits produces. An id outside that
    range is dropped, not sorted (the reference's argsort / bincount path would keep it or raise): the counts exclude it,
    ends[-1] falls short of the number of ids, and the last entries of sorted_expert_idxs / sorted_scattered_idxs and
    the row_slot entries nobody owns stay unwritten. validate=True checks ends[-1] against the number of ids and raises
    on a mismatch; it costs a device-to-host read, so the layer does not ask for it."""
    assert expert_ids.dtype in (torch.int32, torch.long)
    if align is None:
        align = choose_align(expert_ids.numel(), num_experts)
    if is_tracing():
        return _ops.sort_by_expert_segments(expert_ids, num_experts, align)
    seg = _sort_by_expert_eager(expert_ids, num_experts, align)
    if validate and expert_ids.numel() > 0:
        placed = int(seg.ends[-1])
        if placed != expert_ids.numel():
            raise ValueError(
                f"sort_by_expert: {expert_ids.numel() - placed} of {expert_ids.numel()} expert ids lie outside [0, {num_experts})"
            )
    return seg


def _sort_by_expert_eager(expert_ids: torch.Tensor, num_experts: int, align: int) -> ExpertSegments:
    _C.require_gpu(expert_ids)
    ids = expert_ids.contiguous().view(-1)
    R = ids.numel()
    lib = _C.lib()
    dev = ids.device
    max_rows = lib.ck_sort_max_rows(R, num_experts, align)
    i32 = dict(dtype=torch.int32, device=dev)
    u32 = dict(dtype=torch.uint32, device=dev)
    seg = ExpertSegments(
        sorted_expert_idxs=torch.empty(R, **i32),
        sorted_scattered_idxs=torch.empty(R, **i32),
        counts=torch.empty(num_experts, **u32),
        ends=torch.empty(num_experts, **u32),
        starts=torch.empty(num_experts, **u32),
        seg_starts=torch.empty(num_experts + 1, **i32),
        row_slot=torch.empty(max(max_rows, 1), **i32),
        tile_expert=torch.empty(max(max_rows // align, 1), **i32),
        max_rows=max_rows,
        num_experts=num_experts,
        align=align,
    )
    ws = _C.zero_workspace(dev, lib.ck_sort_workspace_words(R, num_experts), "sort")
    with torch.cuda.device(dev):
        _C.check(
            lib.ck_sort_by_expert(
                _C.ptr(ids), int(ids.dtype == torch.long), R, num_experts, align, _C.ptr(seg.sorted_expert_idxs),
                _C.ptr(seg.sorted_scattered_idxs), _C.ptr(seg.counts), _C.ptr(seg.ends), _C.ptr(seg.starts),
                _C.ptr(seg.seg_starts), _C.ptr(seg.row_slot), _C.ptr(seg.tile_expert), _C.ptr(ws), _C.stream(),
            )
        )
    return seg


# ---------------------------------------------------------------------------------------------------------------
# thin launch helpers (allocate outputs, pass pointers)
# ---------------------------------------------------------------------------------------------------------------
class LaunchTimer:
    """Optional per-launch timing of the grouped GEMMs with events on the launch stream (used by bench.py).
    records: list of (kernel name, [N, K] or [M, N] of the launch, start event, end event). Names follow the entry point
    and epilogue, so that at the benchmark's shapes one name is one kernel instantiation: grouped_gemm<epilogue>
    (ck_grouped_gemm), grouped_gemm_nn<epilogue> (ck_grouped_gemm_nn, weights read as stored), grouped_gemm<dw>
    (ck_grouped_gemm_dw, transposed operands), grouped_gemm_dw_rows (ck_grouped_gemm_dw_rows, row-major operands)."""

    def __init__(self) -> None:
        self.records: list = []

    def time(self, name: str, dims: tuple, fn) -> None:
        start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        start.record()
        fn()
        end.record()
        self.records.append((name, dims, start, end))


launch_timer: LaunchTimer | None = None

_EPILOGUE_NAMES = {
    _C.CK_EPI_GROUPED: "grouped_gemm<grouped>",
    _C.CK_EPI_SCATTER: "grouped_gemm<scatter>",
    _C.CK_EPI_SWIGLU: "grouped_gemm<swiglu>",
    _C.CK_EPI_SWIGLU_BWD: "grouped_gemm<swiglu_bwd>",
    _C.CK_EPI_GLU: "grouped_gemm<swiglu>",
    _C.CK_EPI_GELU_TANH: "grouped_gemm<grouped>",
}


_split_workspaces: dict = {}


def _split_workspace(device: torch.device) -> torch.Tensor:
    """Workspace of ck_grouped_gemm_ws / ck_grouped_gemm_nn_ws (split last round of tiles): one buffer per device and
    stream (launches that may overlap must not share one; it needs no initial contents)."""
    if not options.gemm_split:
        return None
    key = (device.index, torch.cuda.current_stream(device).cuda_stream)
    ws = _split_workspaces.get(key)
    if ws is None:
        ws = _split_workspaces[key] = torch.empty(_C.lib().ck_grouped_gemm_workspace_bytes(), dtype=torch.uint8, device=device)
    return ws


def _gemm_f32(a, gather_div, w, w_is_kn: bool, N: int, K: int, seg: ExpertSegments, scatter: bool, y, bias=None,
              rows_in=None, rows_out=None):
    """The grouped GEMMs of fp32 tensors (fp32 MFMA; see ck_grouped_gemm_f32)."""
    cs = seg.c_struct(rows_in, rows_out)
    with torch.cuda.device(w.device):
        _C.check(
            _C.lib().ck_grouped_gemm_f32(
                _C.ptr(a), gather_div, _C.ptr(w), int(w_is_kn), N, K, ctypes.byref(cs), int(scatter), _C.ptr(y), _C.ptr(bias),
                _C.stream(),
            )
        )


def _gemm(a, gather_div, w, seg: ExpertSegments, epilogue, y, y_t=None, aux=None, aux_in=None, rows_in=None, rows_out=None):
    E, N, K = w.shape
    if w.dtype == torch.float32:
        assert epilogue in (_C.CK_EPI_GROUPED, _C.CK_EPI_SCATTER) and y_t is None and aux is None
        return _gemm_f32(a, gather_div, w, False, N, K, seg, epilogue == _C.CK_EPI_SCATTER, y, aux_in, rows_in, rows_out)
    cs = seg.c_struct(rows_in, rows_out)
    if gather_div > 0:  # gathered rows are addressed with 32-bit byte offsets from the start of `a` (the library is not
        # told how many rows `a` has, so this limit is checked here)
        assert a.numel() * a.element_size() < 2**32, "the token-order input of a grouped GEMM must stay below 4 GiB"

    def launch():
        with torch.cuda.device(w.device):
            ws = _split_workspace(w.device) if epilogue in (_C.CK_EPI_GROUPED, _C.CK_EPI_SCATTER) else None
            _C.check(
                _C.lib().ck_grouped_gemm_ws(
                    _C.ptr(a), gather_div, _C.ptr(w), N, K, ctypes.byref(cs), epilogue, _C.ptr(y), _C.ptr(y_t), seg.ld_t,
                    _C.ptr(aux), _C.ptr(aux_in), _C.dtype_code(w.dtype), _C.stream(), _C.ptr(ws), 0 if ws is None else ws.numel(),
                )
            )

    if launch_timer is None:
        launch()
    else:
        launch_timer.time(_EPILOGUE_NAMES[epilogue], (N, K), launch)


def _bias_in_epilogue(seg: ExpertSegments, K: int) -> bool:
    """Whether ck_grouped_gemm takes the per-expert bias as an operand of its grouped / scatter epilogue (the bias joins
    the fp32 accumulators and the output is rounded once, like F.linear). options.bias_fused = False adds it with its
    own kernel after the GEMM instead (two roundings; kept for comparison)."""
    return options.bias_fused


def _fp32(t: torch.Tensor) -> bool:
    """fp32 expert tensors: always the row-major weight-gradient form and the bias in the GEMM's epilogue (the fp32
    kernels have no other form)."""
    return t.dtype == torch.float32


def _gemm_dx(d_y, w, seg: ExpertSegments, epilogue, out, rows_out=None):
    """out = d_y @ w[e] per expert, w [E, out_features, in_features] as the forward stores it: the input-gradient GEMM.
    Reads w contraction-strided where the kernel for that exists (256-row tiles, out_features % 64 == 0); otherwise
    through a transposed copy. rows_out: the table a scatter epilogue writes through (default seg.row_slot)."""
    E, n_out, n_in = w.shape
    if w.dtype == torch.float32:
        return _gemm_f32(d_y, 0, w, True, n_in, n_out, seg, epilogue == _C.CK_EPI_SCATTER, out, None, None, rows_out)
    if seg.align == 256 and n_out % 64 == 0 and options.gemm_nn:
        cs = seg.c_struct(None, rows_out)

        def launch():
            with torch.cuda.device(w.device):
                ws = _split_workspace(w.device)
                _C.check(
                    _C.lib().ck_grouped_gemm_nn_ws(
                        _C.ptr(d_y), _C.ptr(w), n_in, n_out, ctypes.byref(cs), epilogue, _C.ptr(out), _C.dtype_code(w.dtype),
                        _C.stream(), _C.ptr(ws), 0 if ws is None else ws.numel(),
                    )
                )

        if launch_timer is None:
            launch()
        else:
            launch_timer.time(_EPILOGUE_NAMES[epilogue].replace("grouped_gemm<", "grouped_gemm_nn<"), (n_in, n_out), launch)
        return
    _gemm(d_y, 0, _transpose_weights(w), seg, epilogue, out, rows_out=rows_out)


def _gemm_dw(a_t, b_t, seg: ExpertSegments, dw):
    E, M, N = dw.shape
    cs = seg.c_struct()

    def launch():
        with torch.cuda.device(dw.device):
            _C.check(
                _C.lib().ck_grouped_gemm_dw(
                    _C.ptr(a_t), _C.ptr(b_t), seg.ld_t, M, N, ctypes.byref(cs), _C.ptr(dw), _C.dtype_code(dw.dtype),
                    _C.stream(),
                )
            )

    if launch_timer is None:
        launch()
    else:
        launch_timer.time("grouped_gemm<dw>", (M, N), launch)


def _gemm_dw_rows(a, b, seg: ExpertSegments, dw):
    """dw[e] = a[rows of e]^T @ b[rows of e] from row-major padded-grouped operands (no transposed copies)."""
    E, M, N = dw.shape
    cs = seg.c_struct()
    if dw.dtype == torch.float32:
        with torch.cuda.device(dw.device):
            _C.check(_C.lib().ck_grouped_gemm_dw_f32(_C.ptr(a), _C.ptr(b), M, N, ctypes.byref(cs), _C.ptr(dw), _C.stream()))
        return

    def launch():
        with torch.cuda.device(dw.device):
            _C.check(
                _C.lib().ck_grouped_gemm_dw_rows(
                    _C.ptr(a), _C.ptr(b), M, N, ctypes.byref(cs), _C.ptr(dw), _C.dtype_code(dw.dtype), _C.stream()
                )
            )

    if launch_timer is None:
        launch()
    else:
        launch_timer.time("grouped_gemm_dw_rows", (M, N), launch)


def _dw_from_rows(max_rows: int, num_experts: int, align: int, *shapes: tuple[int, int]) -> bool:
    """Whether the weight-gradient GEMMs of shapes (M, N), ... read row-major operands (ck_grouped_gemm_dw_rows) instead
    of transposed copies: whenever that kernel takes the shapes. Not writing (and not holding) the transposes outweighs
    the 384-wide tiles the transposed form can use (measured: fine-grained layer 4 % faster, Mixtral-shape layer 0.4 %).
    A function of sizes only, so that forward, backward and the traced (fake) implementations agree on which tensors
    exist."""
    return options.dw_rows and align % 64 == 0 and all(min(m, n) >= 256 and m % 8 == 0 and n % 8 == 0 for m, n in shapes)


def _group_rows(src, coeff, fan_out, seg: ExpertSegments, want_grouped: bool, want_transposed: bool, rows=None):
    """Padded grouped copy of `src` rows (fan_out == 0: src is already padded-grouped) and / or its transpose. rows: the
    table the rows are read through (default seg.row_slot)."""
    H = src.size(-1)
    grouped = torch.empty(seg.max_rows, H, dtype=src.dtype, device=src.device) if want_grouped else None
    grouped_t = torch.empty(H, seg.ld_t, dtype=src.dtype, device=src.device) if want_transposed else None
    with torch.cuda.device(src.device):
        _C.check(
            _C.lib().ck_group_rows_padded(
                _C.ptr(src), _C.ptr(coeff), fan_out, H, _C.ptr(seg.row_slot if rows is None else rows), _C.ptr(seg.seg_starts), _C.ptr(seg.counts),
                _C.ptr(seg.tile_expert), seg.align, seg.max_rows, _C.ptr(grouped), _C.ptr(grouped_t), seg.ld_t,
                _C.dtype_code(src.dtype), _C.stream(),
            )
        )
    return grouped, grouped_t


def _transpose_weights(w: torch.Tensor) -> torch.Tensor:
    E, N, K = w.shape
    w_t = torch.empty(E, K, N, dtype=w.dtype, device=w.device)
    with torch.cuda.device(w.device):
        _C.check(_C.lib().ck_transpose_batched(_C.ptr(w), E, N, K, _C.ptr(w_t), _C.dtype_code(w.dtype), _C.stream()))
    return w_t


def _combine(expanded, gates, T, k, H, grad_out=None, want_out=True, want_d_gates=False):
    out = torch.empty(T, H, dtype=expanded.dtype, device=expanded.device) if want_out else None
    d_gates = torch.empty(T, k, dtype=expanded.dtype, device=expanded.device) if want_d_gates else None
    with torch.cuda.device(expanded.device):
        _C.check(
            _C.lib().ck_combine_rows(
                _C.ptr(expanded), _C.ptr(gates), T, k, H, _C.ptr(out), _C.ptr(grad_out), _C.ptr(d_gates),
                _C.dtype_code(expanded.dtype), _C.stream(),
            )
        )
    return out, d_gates


def _gate_grad(expanded, grad_out, T, k, H, gates_dtype, slot):
    """d_gates in fp32 (kept in `slot` for the router's backward) and rounded to the gates' dtype for autograd."""
    d32 = torch.empty(T, k, dtype=torch.float32, device=expanded.device)
    with torch.cuda.device(expanded.device):
        _C.check(
            _C.lib().ck_gate_grad_f32(
                _C.ptr(expanded), _C.ptr(grad_out), T, k, H, _C.ptr(d32), _C.dtype_code(expanded.dtype), _C.stream()
            )
        )
    if slot is not None:
        slot.d_gates_f32 = d32
    return d32.to(gates_dtype)


def gather_rows(src: torch.Tensor, idx: torch.Tensor, coeff: torch.Tensor | None = None, fan_out: int = 1) -> torch.Tensor:
    """out[n] = src[idx[n] // fan_out] * coeff[idx[n]] -- the reference's `group` (ops.py:108-140)."""
    _C.require_gpu(src, idx)
    src = src.contiguous()
    out = torch.empty(idx.numel(), src.size(-1), dtype=src.dtype, device=src.device)
    with torch.cuda.device(src.device):
        _C.check(
            _C.lib().ck_gather_rows(
                _C.ptr(src), _C.ptr(idx), _C.ptr(coeff), fan_out, idx.numel(), src.size(-1), _C.ptr(out),
                _C.dtype_code(src.dtype), _C.stream(),
            )
        )
    return out


def _add_expert_bias(y: torch.Tensor, bias: torch.Tensor, seg: ExpertSegments, row_expert: torch.Tensor | None) -> None:
    """y[r] += bias[expert of row r] in place: padded grouped rows (row_expert None) or token-order rows."""
    cs = seg.c_struct()
    with torch.cuda.device(y.device):
        _C.check(
            _C.lib().ck_add_expert_bias(
                _C.ptr(y), y.size(0), y.size(1), _C.ptr(bias), _C.ptr(row_expert), None if row_expert is not None else ctypes.byref(cs),
                _C.dtype_code(y.dtype), _C.stream(),
            )
        )


def _expert_bias_grad(d_y: torch.Tensor, seg: ExpertSegments) -> torch.Tensor:
    """[E, N] column sums of the padded grouped rows of every expert."""
    d_bias = torch.empty(seg.num_experts, d_y.size(1), dtype=d_y.dtype, device=d_y.device)
    cs = seg.c_struct()
    with torch.cuda.device(d_y.device):
        _C.check(
            _C.lib().ck_expert_bias_grad(
                _C.ptr(d_y), d_y.size(1), ctypes.byref(cs), _C.ptr(d_bias), _C.dtype_code(d_y.dtype), _C.stream()
            )
        )
    return d_bias


def _slot_experts(seg: ExpertSegments) -> torch.Tensor:
    """Expert of every flat (token, slot) index, int32 [R] (the inverse of the sort)."""
    slot_expert = torch.empty_like(seg.sorted_expert_idxs)
    slot_expert[seg.sorted_scattered_idxs.long()] = seg.sorted_expert_idxs
    return slot_expert


def _check_expert_dtypes(x: torch.Tensor, *weights: torch.Tensor) -> None:
    if x.dtype not in (torch.bfloat16, torch.float16, torch.float32):
        raise NotImplementedError(f"the MI355X expert GEMMs take bf16 / fp16 / fp32 inputs; got {x.dtype}")
    for w in weights:
        assert w.dtype == x.dtype, "expert weights and activations should have the same dtype"
    assert x.size(-1) % 8 == 0, "hidden size should be a multiple of 8"


# ---------------------------------------------------------------------------------------------------------------
# generic expert linears (any activation between them)
# ---------------------------------------------------------------------------------------------------------------
class _ExpertsUp(torch.autograd.Function):
    """x [T, H] (token order) -> y [max_rows, N] (padded grouped): the reference's c_fc with grouped_out=True.
    gelu=True: returns gelu_tanh(y) instead, computed in the GEMM's epilogue from the rounded y (the activation module
    applied to y would read the same values); y is kept for the backward pass only."""

    @staticmethod
    def forward(ctx, x, w, seg: ExpertSegments, k: int, bias=None, gelu: bool = False):
        x = x.contiguous()
        w = w.contiguous()
        E, N, K = w.shape
        # pad rows are never written by the kernel; zeros keep any activation applied on top finite
        y = torch.zeros(seg.max_rows, N, dtype=x.dtype, device=x.device)
        act = torch.zeros_like(y) if gelu else None
        fused_bias = bias is not None and (gelu or _fp32(x) or _bias_in_epilogue(seg, K))
        _gemm(x, k, w, seg, _C.CK_EPI_GELU_TANH if gelu else _C.CK_EPI_GROUPED, y, aux=act,
              aux_in=bias.contiguous() if fused_bias else None)
        if bias is not None and not fused_bias:
            _add_expert_bias(y, bias.contiguous(), seg, None)
        ctx.gelu = gelu
        if gelu:
            ctx.save_for_backward(x, w, y)
        else:
            ctx.save_for_backward(x, w)
        ctx.seg, ctx.k = seg, k
        return act if gelu else y

    @staticmethod
    def backward(ctx, d_y):
        x, w = ctx.saved_tensors[:2]
        seg, k = ctx.seg, ctx.k
        T, K = x.shape
        d_y = d_y.contiguous()
        if getattr(ctx, "gelu", False):  # d_y arrives as d_act: through the activation first
            pre, d_act = ctx.saved_tensors[2], d_y
            d_y = torch.empty_like(d_act)
            with torch.cuda.device(d_act.device):
                _C.check(_C.lib().ck_gelu_tanh_bwd(_C.ptr(pre), _C.ptr(d_act), _C.ptr(d_y), d_act.numel(),
                                                   _C.dtype_code(d_act.dtype), _C.stream()))
        d_x = d_w = d_bias = None
        if len(ctx.needs_input_grad) > 4 and ctx.needs_input_grad[4]:
            d_bias = _expert_bias_grad(d_y, seg)
        if ctx.needs_input_grad[1]:
            d_w = torch.empty_like(w)
            if _fp32(x) or _dw_from_rows(seg.max_rows, seg.num_experts, seg.align, tuple(w.shape[1:])):
                x_g, _ = _group_rows(x, None, k, seg, True, False)
                _gemm_dw_rows(d_y, x_g, seg, d_w)
            else:
                _, d_y_t = _group_rows(d_y, None, 0, seg, False, True)
                _, x_t = _group_rows(x, None, k, seg, False, True)
                _gemm_dw(d_y_t, x_t, seg, d_w)
        if ctx.needs_input_grad[0]:
            d_expanded = torch.empty(T * k, K, dtype=x.dtype, device=x.device)
            _gemm_dx(d_y, w, seg, _C.CK_EPI_SCATTER, d_expanded)
            d_x = d_expanded if k == 1 else _combine(d_expanded, None, T, k, K)[0]
        return d_x, d_w, None, None, d_bias, None


class _ExpertsDown(torch.autograd.Function):
    """h [max_rows, I] (padded grouped), gates [T, k] -> out [T, H]: the reference's c_proj with grouped_in=True."""

    @staticmethod
    def forward(ctx, h, w, gates, seg: ExpertSegments, bias=None, slot_expert=None, gate_slot=None):
        ctx.gate_slot = gate_slot
        h = h.contiguous()
        w = w.contiguous()
        gates = gates.contiguous()
        T, k = gates.shape
        E, N, K = w.shape
        expanded = torch.empty(T * k, N, dtype=h.dtype, device=h.device)
        fused_bias = bias is not None and (_fp32(h) or _bias_in_epilogue(seg, K))
        _gemm(h, 0, w, seg, _C.CK_EPI_SCATTER, expanded, aux_in=bias.contiguous() if fused_bias else None)
        if bias is not None and not fused_bias:  # before the gate multiply, as torch_implementation.py:160-163
            _add_expert_bias(expanded, bias.contiguous(), seg, slot_expert if slot_expert is not None else _slot_experts(seg))
        out, _ = _combine(expanded, gates, T, k, N)
        ctx.save_for_backward(h, w, gates, expanded)
        ctx.seg = seg
        return out

    @staticmethod
    def backward(ctx, grad_out):
        h, w, gates, expanded = ctx.saved_tensors
        seg = ctx.seg
        T, k = gates.shape
        E, N, K = w.shape
        grad_out = grad_out.contiguous()
        d_h = d_w = d_gates = d_bias = None
        if ctx.needs_input_grad[2]:
            d_gates = _gate_grad(expanded, grad_out, T, k, N, gates.dtype, ctx.gate_slot)
        need_w = ctx.needs_input_grad[1]
        rows_form = _fp32(h) or _dw_from_rows(seg.max_rows, seg.num_experts, seg.align, (N, K))
        d_y, d_y_t = _group_rows(grad_out, gates, k, seg, True, need_w and not rows_form)
        if len(ctx.needs_input_grad) > 4 and ctx.needs_input_grad[4]:
            d_bias = _expert_bias_grad(d_y, seg)  # d_y: the gate-scaled grad_out rows in padded grouped order
        if need_w:
            d_w = torch.empty_like(w)
            if rows_form:
                _gemm_dw_rows(d_y, h, seg, d_w)
            else:
                _, h_t = _group_rows(h, None, 0, seg, False, True)
                _gemm_dw(d_y_t, h_t, seg, d_w)
        if ctx.needs_input_grad[0]:
            d_h = torch.zeros(seg.max_rows, K, dtype=h.dtype, device=h.device)
            _gemm_dx(d_y, w, seg, _C.CK_EPI_GROUPED, d_h)
        return d_h, d_w, d_gates, None, d_bias, None, None


def experts_up(
    x: torch.Tensor, weight: torch.Tensor, seg: ExpertSegments, k: int, bias: torch.Tensor | None = None,
    gelu_tanh: bool = False,
) -> torch.Tensor:
    """x [T, H] -> c_fc output in padded grouped order [max_rows, N] (+ bias[e] on expert e's rows); with gelu_tanh, the
    tanh-approximated GELU of that output, applied in the GEMM's epilogue."""
    _check_expert_dtypes(x, weight)
    assert bias is None or (bias.dtype == x.dtype and bias.shape == weight.shape[:2]), "bias should be [E, out] in x.dtype"
    if is_tracing():
        op = _ops.experts_up_gelu if gelu_tanh else _ops.experts_up
        out = op(
            x, weight, bias, seg.seg_starts, seg.counts, seg.tile_expert, seg.row_slot, seg.max_rows, seg.num_experts,
            seg.align, k,
        )
        return out[0] if gelu_tanh else out
    _C.require_gpu(x, weight, bias)
    return _ExpertsUp.apply(x, weight, seg, k, bias, gelu_tanh)


def experts_down(
    h: torch.Tensor, weight: torch.Tensor, gates: torch.Tensor, seg: ExpertSegments, bias: torch.Tensor | None = None
) -> torch.Tensor:
    """h [max_rows, I] (padded grouped) -> sum_k gates * (c_proj output + bias[e]) in token order [T, N]."""
    _check_expert_dtypes(h, weight)
    assert bias is None or (bias.dtype == h.dtype and bias.shape == weight.shape[:2]), "bias should be [E, out] in h.dtype"
    if is_tracing():
        slot_expert = _slot_experts(seg) if bias is not None else None
        return _ops.experts_down(
            h, weight, gates.to(h.dtype), bias, slot_expert, seg.seg_starts, seg.counts, seg.tile_expert, seg.row_slot,
            seg.max_rows, seg.num_experts, seg.align,
        )[0]
    _C.require_gpu(h, weight, gates, bias)
    return _ExpertsDown.apply(h, weight, gates.to(h.dtype), seg, bias, None, _gate_slot(gates))


# ---------------------------------------------------------------------------------------------------------------
# fused SwiGLU expert block
# ---------------------------------------------------------------------------------------------------------------
class _SwigluExperts(torch.autograd.Function):
    """out = combine_k( gates * c_proj( swiglu_packed( c_fc(x) ) ) ) with the SwiGLU forward fused into the c_fc
    epilogue and the SwiGLU backward fused into the epilogue of the c_proj input-gradient GEMM."""

    @staticmethod
    def forward(ctx, x, w_fc, w_proj, gates, seg: ExpertSegments, act_kind: int = _C.CK_ACT_SWIGLU, gate_slot=None):
        ctx.gate_slot = gate_slot
        x = x.contiguous()
        w_fc = w_fc.contiguous()
        w_proj = w_proj.contiguous()
        gates = gates.contiguous()
        T, H = x.shape
        k = gates.size(1)
        E, two_i, _ = w_fc.shape
        I = two_i // 2
        dev, dt = x.device, x.dtype
        need_grad = any(ctx.needs_input_grad[:4])

        pre = torch.empty(seg.max_rows, two_i, dtype=dt, device=dev)
        act = torch.empty(seg.max_rows, I, dtype=dt, device=dev)
        # d_w_proj needs the activation: transposed (written by the same epilogue) or, in the row-major form, as it is
        rows_form = _dw_from_rows(seg.max_rows, seg.num_experts, seg.align, (H, I), (two_i, H))
        act_t = torch.empty(I, seg.ld_t, dtype=dt, device=dev) if ctx.needs_input_grad[2] and not rows_form else None
        _gemm(x, k, w_fc, seg, _C.CK_EPI_GLU if act_kind == _C.CK_ACT_GLU else _C.CK_EPI_SWIGLU, pre, y_t=act_t, aux=act)

        expanded = torch.empty(T * k, H, dtype=dt, device=dev)
        _gemm(act, 0, w_proj, seg, _C.CK_EPI_SCATTER, expanded)
        out, _ = _combine(expanded, gates, T, k, H)

        if need_grad:
            act_saved = (act if ctx.needs_input_grad[2] else None) if rows_form else act_t
            ctx.save_for_backward(x, w_fc, w_proj, gates, pre, act_saved, expanded)
        ctx.seg, ctx.act_kind = seg, act_kind
        return out

    @staticmethod
    def backward(ctx, grad_out):
        x, w_fc, w_proj, gates, pre, act_saved, expanded = ctx.saved_tensors
        seg, act_kind = ctx.seg, ctx.act_kind
        T, H = x.shape
        k = gates.size(1)
        E, two_i, _ = w_fc.shape
        I = two_i // 2
        dev, dt = x.device, x.dtype
        grad_out = grad_out.contiguous()
        need_x, need_fc, need_proj, need_gates = ctx.needs_input_grad[:4]
        d_x = d_w_fc = d_w_proj = d_gates = None
        rows_form = _dw_from_rows(seg.max_rows, seg.num_experts, seg.align, (H, I), (two_i, H))  # as in forward

        if need_gates:
            d_gates = _gate_grad(expanded, grad_out, T, k, H, gates.dtype, ctx.gate_slot)

        # gate-scaled grad_out rows in padded grouped order (+ transpose for d_w_proj unless it reads rows)
        d_y, d_y_t = _group_rows(grad_out, gates, k, seg, True, need_proj and not rows_form)
        if need_proj:
            d_w_proj = torch.empty_like(w_proj)
            if rows_form:
                _gemm_dw_rows(d_y, act_saved, seg, d_w_proj)
            else:
                _gemm_dw(d_y_t, act_saved, seg, d_w_proj)
            del d_y_t

        if need_x or need_fc:
            # d_act = d_y @ w_proj with the leanest epilogue, then one streaming pass for the SwiGLU backward and the
            # transpose d_w_fc needs. (The GEMM can also do this in its epilogue, CK_EPI_SWIGLU_BWD, but with one
            # workgroup per CU the epilogue is time the MFMA units idle, while the streaming pass runs at HBM speed.)
            d_act = torch.empty(seg.max_rows, I, dtype=dt, device=dev)
            _gemm_dx(d_y, w_proj, seg, _C.CK_EPI_GROUPED, d_act)
            del d_y
            d_pre = torch.empty(seg.max_rows, two_i, dtype=dt, device=dev)
            d_pre_t = torch.empty(two_i, seg.ld_t, dtype=dt, device=dev) if need_fc and not rows_form else None
            with torch.cuda.device(dev):
                _C.check(
                    _C.lib().ck_swiglu_bwd_grouped(
                        _C.ptr(pre), _C.ptr(d_act), I, _C.ptr(seg.seg_starts), _C.ptr(seg.counts), _C.ptr(seg.tile_expert),
                        seg.align, seg.max_rows, _C.ptr(d_pre), _C.ptr(d_pre_t), seg.ld_t, act_kind, _C.dtype_code(dt),
                        _C.stream(),
                    )
                )
            del d_act
            if need_fc:
                d_w_fc = torch.empty_like(w_fc)
                if rows_form:
                    x_g, _ = _group_rows(x, None, k, seg, True, False)
                    _gemm_dw_rows(d_pre, x_g, seg, d_w_fc)
                    del x_g
                else:
                    _, x_t = _group_rows(x, None, k, seg, False, True)
                    _gemm_dw(d_pre_t, x_t, seg, d_w_fc)
                    del d_pre_t, x_t
            if need_x:
                d_expanded = torch.empty(T * k, H, dtype=dt, device=dev)
                _gemm_dx(d_pre, w_fc, seg, _C.CK_EPI_SCATTER, d_expanded)
                d_x = d_expanded if k == 1 else _combine(d_expanded, None, T, k, H)[0]
        return d_x, d_w_fc, d_w_proj, d_gates, None, None, None


def swiglu_experts(
    x: torch.Tensor, w_fc: torch.Tensor, w_proj: torch.Tensor, gates: torch.Tensor, seg: ExpertSegments,
    act_kind: int = _C.CK_ACT_SWIGLU,
) -> torch.Tensor:
    """Fused expert block for `is_glu=True` (c_fc columns [up | gate]) with `activation_function = swiglu_packed_cute`
    (act_kind CK_ACT_SWIGLU: up * silu(gate)) or `torch.nn.GLU()` (CK_ACT_GLU: up * sigmoid(gate))."""
    _check_expert_dtypes(x, w_fc, w_proj)
    assert x.dtype != torch.float32, "the fused expert block is 16-bit; fp32 layers run experts_up -> activation -> experts_down"
    assert w_fc.size(1) % 16 == 0, "intermediate size should be a multiple of 8"
    if is_tracing():
        grad = torch.is_grad_enabled()
        return _ops.swiglu_experts(
            x, w_fc, w_proj, gates.to(x.dtype), seg.seg_starts, seg.counts, seg.tile_expert, seg.row_slot, seg.max_rows,
            seg.num_experts, seg.align, grad and x.requires_grad, grad and w_fc.requires_grad,
            grad and w_proj.requires_grad, grad and gates.requires_grad, act_kind,
        )[0]
    _C.require_gpu(x, w_fc, w_proj, gates)
    return _SwigluExperts.apply(x, w_fc, w_proj, gates.to(x.dtype), seg, act_kind, _gate_slot(gates))


# ---------------------------------------------------------------------------------------------------------------
# the reference's own expert-linear interface: three index tensors, unpadded grouped rows
# ---------------------------------------------------------------------------------------------------------------
def bincount(x: torch.Tensor, minlength: int) -> torch.Tensor:
    """Histogram of expert ids as the reference's helper returns it (triton_implementation/ops.py:19-28): int64 counts,
    computed by the count kernel (ids outside [0, minlength) are not counted, where torch.bincount would grow or raise)."""
    from .continuous_count import continuous_count_cute

    return continuous_count_cute(x.reshape(-1), minlength).to(torch.int64)


_segments_cache: list = []  # [(sorted_expert_idxs, sorted_scattered_idxs, expert_offsets, versions, align, ExpertSegments)]


@torch.no_grad()
def segments_from_sorted(
    sorted_expert_idxs: torch.Tensor, sorted_scattered_idxs: torch.Tensor, expert_offsets: torch.Tensor,
    align: int | None = None,
) -> ExpertSegments:
    """The padded grouped layout for a sort the caller did: (sorted_expert_idxs, sorted_scattered_idxs) =
    selected_experts.flatten().sort() and expert_offsets = bincount(...).cumsum(-1), the arguments of the reference's
    expert linears (triton_implementation/__init__.py:82-83). One small launch; the result for the last two distinct
    argument triples is kept, so that c_fc and c_proj of one layer call share it."""
    _C.require_gpu(sorted_expert_idxs, sorted_scattered_idxs, expert_offsets)
    assert sorted_expert_idxs.dim() == 1 and sorted_expert_idxs.shape == sorted_scattered_idxs.shape
    assert sorted_expert_idxs.dtype == sorted_scattered_idxs.dtype and sorted_expert_idxs.dtype in (torch.int32, torch.long)
    assert expert_offsets.dim() == 1 and expert_offsets.dtype in (torch.int32, torch.uint32, torch.long)
    R, E = sorted_expert_idxs.numel(), expert_offsets.numel()
    if align is None:
        align = choose_align(R, E)
    tensors = (sorted_expert_idxs, sorted_scattered_idxs, expert_offsets)
    versions = tuple(t._version for t in tensors)
    for entry in _segments_cache:
        if all(a is b for a, b in zip(entry[0], tensors)) and entry[1] == versions and entry[2] == align:
            return entry[3]
    se, ss, off = (t.contiguous() for t in tensors)
    lib = _C.lib()
    dev = se.device
    max_rows = lib.ck_sort_max_rows(R, E, align)
    i32 = dict(dtype=torch.int32, device=dev)
    seg = ExpertSegments(
        sorted_expert_idxs=se, sorted_scattered_idxs=ss, counts=torch.empty(E, dtype=torch.uint32, device=dev), ends=off,
        starts=None, seg_starts=torch.empty(E + 1, **i32), row_slot=torch.empty(max(max_rows, 1), **i32),
        tile_expert=torch.empty(max(max_rows // align, 1), **i32), max_rows=max_rows, num_experts=E, align=align,
        row_pos=torch.empty(max(max_rows, 1), **i32),
    )
    with torch.cuda.device(dev):
        _C.check(
            lib.ck_segments_from_sorted(
                _C.ptr(se), _C.ptr(ss), int(se.dtype == torch.long), _C.ptr(off), int(off.dtype == torch.long), R, E, align,
                _C.ptr(seg.counts), _C.ptr(seg.seg_starts), _C.ptr(seg.row_slot), _C.ptr(seg.row_pos), _C.ptr(seg.tile_expert),
                _C.stream(),
            )
        )
    _segments_cache.insert(0, (tensors, versions, align, seg))
    del _segments_cache[2:]
    return seg


class _ScatteredExperts(torch.autograd.Function):
    """One expert linear on the reference's index tensors (triton_implementation/ops.py:143-292), w [E, N, K] as the
    module stores it. Input rows: token order [T, K] read through sorted_scattered_idxs // k, or (grouped_in) unpadded
    grouped rows [R, K] in sorted order. Output: [R, N] in (token, slot) order, or (grouped_out) in sorted order, or
    (gates [T, fan]) the gated sum over a token's slots [T, N]. The GEMM runs on the padded layout and reads / writes the
    caller's rows through the row tables, so no padded copy of the input or output is made in the forward pass."""

    @staticmethod
    def forward(ctx, x, w, k, sorted_expert_idxs, sorted_scattered_idxs, expert_offsets, gates, grouped_in, grouped_out,
                bias=None, gate_slot=None):
        assert not (gates is not None and grouped_out), "gated outputs are combined per token, not grouped"
        seg = segments_from_sorted(sorted_expert_idxs, sorted_scattered_idxs, expert_offsets)
        x = x.contiguous()
        w = w.contiguous()
        E, N, K = w.shape
        R = sorted_expert_idxs.numel()
        assert x.size(-1) == K and x.size(0) == (R if grouped_in else R // k), "input rows do not match the index tensors"
        out = torch.empty(R, N, dtype=x.dtype, device=x.device)
        ctx.seg, ctx.k, ctx.grouped_in, ctx.grouped_out, ctx.gate_slot = seg, k, grouped_in, grouped_out, gate_slot
        if R == 0:  # no routed rows: nothing to launch
            ctx.save_for_backward(x, w, gates, None)
            return out if gates is None else torch.zeros(gates.size(0), N, dtype=x.dtype, device=x.device)
        fused_bias = bias is not None and (_fp32(x) or _bias_in_epilogue(seg, K))
        _gemm(
            x, 1 if grouped_in else k, w, seg, _C.CK_EPI_SCATTER, out, aux_in=bias.contiguous() if fused_bias else None,
            rows_in=seg.row_pos if grouped_in else seg.row_slot, rows_out=seg.row_pos if grouped_out else seg.row_slot,
        )
        if bias is not None and not fused_bias:
            row_expert = sorted_expert_idxs.to(torch.int32) if grouped_out else _slot_experts(seg)
            _add_expert_bias(out, bias.contiguous(), seg, row_expert)
        expanded = None
        if gates is not None:
            gates = gates.contiguous()
            T, fan = gates.shape
            assert T * fan == R, "gates do not match the index tensors"
            expanded = out
            out, _ = _combine(expanded, gates, T, fan, N)
        ctx.save_for_backward(x, w, gates, expanded)
        return out

    @staticmethod
    def backward(ctx, grad_out):
        x, w, gates, expanded = ctx.saved_tensors
        seg, k, grouped_in, grouped_out = ctx.seg, ctx.k, ctx.grouped_in, ctx.grouped_out
        E, N, K = w.shape
        grad_out = grad_out.contiguous()
        need = ctx.needs_input_grad
        need_x, need_w, need_gates = need[0], need[1], need[6]
        need_bias = len(need) > 9 and need[9]
        d_x = d_w = d_gates = d_bias = None
        if seg.sorted_expert_idxs.numel() == 0:  # no routed rows: every gradient is zero
            return (
                torch.zeros_like(x) if need_x else None, torch.zeros_like(w) if need_w else None, None, None, None, None,
                torch.zeros_like(gates) if need_gates and gates is not None else None, None, None,
                torch.zeros(E, N, dtype=w.dtype, device=w.device) if need_bias else None, None,
            )
        # the output gradient as padded grouped rows: what both the weight- and the input-gradient GEMM read
        if gates is not None:
            T, fan = gates.shape
            if need_gates:
                d_gates = _gate_grad(expanded, grad_out, T, fan, N, gates.dtype, ctx.gate_slot)
            d_y, _ = _group_rows(grad_out, gates, fan, seg, True, False)
        elif grouped_out:
            d_y, _ = _group_rows(grad_out, None, 1, seg, True, False, rows=seg.row_pos)
        else:
            d_y, _ = _group_rows(grad_out, None, 1, seg, True, False)
        if need_bias:
            d_bias = _expert_bias_grad(d_y, seg)
        if need_w:
            x_g, _ = _group_rows(x, None, 1 if grouped_in else k, seg, True, False, rows=seg.row_pos if grouped_in else None)
            d_w = torch.empty_like(w)
            if _fp32(x) or _dw_from_rows(seg.max_rows, E, seg.align, (N, K)):
                _gemm_dw_rows(d_y, x_g, seg, d_w)
            else:
                _, d_y_t = _group_rows(d_y, None, 0, seg, False, True)
                _, x_t = _group_rows(x_g, None, 0, seg, False, True)
                _gemm_dw(d_y_t, x_t, seg, d_w)
        if need_x:
            R = seg.sorted_expert_idxs.numel()
            d_rows = torch.empty(R, K, dtype=x.dtype, device=x.device)
            _gemm_dx(d_y, w, seg, _C.CK_EPI_SCATTER, d_rows, rows_out=seg.row_pos if grouped_in else seg.row_slot)
            d_x = d_rows if grouped_in or k == 1 else _combine(d_rows, None, x.size(0), k, K)[0]
        return d_x, d_w, None, None, None, None, d_gates, None, None, d_bias, None


def scattered_experts(
    inputs: torch.Tensor, expert_weights: torch.Tensor, k: int, sorted_expert_idxs: torch.Tensor,
    sorted_scattered_idxs: torch.Tensor, expert_offsets: torch.Tensor, gates: torch.Tensor | None = None,
    grouped_in: bool = False, grouped_out: bool = False, bias: torch.Tensor | None = None,
) -> torch.Tensor:
    """The reference's scattered_experts (triton_implementation/ops.py:295-316), same arguments in the same order:
    expert_weights is the [E, in, out] VIEW `weight.permute(0, 2, 1)` of an [E, out, in] parameter (any other layout is
    copied). `bias` [E, out] is this build's addition (the reference's launcher has none and its module drops the bias)."""
    w = expert_weights.permute(0, 2, 1)  # back to the parameter's own layout: no copy when the argument was the view
    _check_expert_dtypes(inputs, w)
    assert bias is None or (bias.dtype == inputs.dtype and bias.shape == w.shape[:2]), "bias should be [E, out] in x.dtype"
    if gates is not None:
        gates_in = gates
        gates = gates.to(inputs.dtype)
    if is_tracing():
        out = _ops.scattered_experts(
            inputs, w, gates, bias, sorted_expert_idxs, sorted_scattered_idxs, expert_offsets, k, grouped_in, grouped_out
        )
        return out[0]
    _C.require_gpu(inputs, w, gates, bias, sorted_expert_idxs, sorted_scattered_idxs, expert_offsets)
    return _ScatteredExperts.apply(
        inputs, w, k, sorted_expert_idxs, sorted_scattered_idxs, expert_offsets, gates, grouped_in, grouped_out, bias,
        _gate_slot(gates_in) if gates is not None else None,
    )
