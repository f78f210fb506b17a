"""ctypes binding of libck_mi355.so (the C ABI declared in include/ck_mi355.h).

The library is built ahead of time by cute-kernels_amd/build.py and lives next to this file. There is no fallback: if it
is missing, or a call is rejected, the caller gets an exception -- never a silent PyTorch path.
"""

from __future__ import annotations

import ctypes
import os
from ctypes import POINTER, Structure, c_char_p, c_float, c_int32, c_int64, c_void_p

import torch


_LIB_NAME = "libck_mi355.so"
_LIB_PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), _LIB_NAME)

CK_F32, CK_F16, CK_BF16 = 0, 1, 2
CK_EPI_GROUPED, CK_EPI_SCATTER, CK_EPI_SWIGLU, CK_EPI_SWIGLU_BWD = 0, 1, 2, 3
CK_EPI_GLU = 5
CK_EPI_GELU_TANH = 6
CK_ACT_SWIGLU, CK_ACT_GLU, CK_ACT_GELU_TANH = 0, 1, 2

_DTYPE_CODES = {torch.float32: CK_F32, torch.float16: CK_F16, torch.bfloat16: CK_BF16}


class ck_segments(Structure):
    _fields_ = [
        ("seg_starts", c_void_p),
        ("counts", c_void_p),
        ("tile_expert", c_void_p),
        ("row_slot", c_void_p),
        ("max_rows", c_int64),
        ("num_experts", c_int32),
        ("align", c_int32),
        ("row_slot_out", c_void_p),
    ]


# name -> (restype, argtypes); mirrors include/ck_mi355.h one to one
_SIGNATURES = {
    "ck_last_error_string": (c_char_p, []),
    "ck_abi_version": (c_int32, []),
    "ck_debug_set_option": (c_int32, [c_char_p, c_int64]),
    "ck_count_workspace_words": (c_int64, [c_int32]),
    "ck_count_offsets": (c_int32, [c_void_p, c_int32, c_int64, c_int32, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p]),
    "ck_count_offsets_static": (c_int32, [c_void_p, c_int32, c_int64, c_int32, c_void_p, c_void_p, c_void_p, c_void_p]),
    "ck_route_topk_softmax": (c_int32, [c_void_p, c_int32, c_int64, c_int32, c_int32, c_void_p, c_void_p, c_void_p, c_void_p]),
    "ck_route_topk_softmax_bwd": (c_int32, [c_void_p, c_void_p, c_void_p, c_int64, c_int32, c_int32, c_void_p, c_int32, c_void_p]),
    "ck_route_topk_softmax_bwd_exact": (c_int32, [c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_int32, c_int32, c_void_p, c_int32, c_void_p]),
    "ck_sort_max_rows": (c_int64, [c_int64, c_int32, c_int32]),
    "ck_sort_workspace_words": (c_int64, [c_int64, c_int32]),
    "ck_sort_by_expert": (c_int32, [c_void_p, c_int32, c_int64, c_int32, c_int32] + [c_void_p] * 10),
    "ck_segments_from_sorted": (
        c_int32,
        [c_void_p, c_void_p, c_int32, c_void_p, c_int32, c_int64, c_int32, c_int32, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p],
    ),
    "ck_gather_rows": (c_int32, [c_void_p, c_void_p, c_void_p, c_int32, c_int64, c_int32, c_void_p, c_int32, c_void_p]),
    "ck_combine_rows": (c_int32, [c_void_p, c_void_p, c_int64, c_int32, c_int32, c_void_p, c_void_p, c_void_p, c_int32, c_void_p]),
    "ck_gate_grad_f32": (c_int32, [c_void_p, c_void_p, c_int64, c_int32, c_int32, c_void_p, c_int32, c_void_p]),
    "ck_group_rows_padded": (
        c_int32,
        [c_void_p, c_void_p, c_int32, c_int32, c_void_p, c_void_p, c_void_p, c_void_p, c_int32, c_int64, c_void_p, c_void_p, c_int64, c_int32, c_void_p],
    ),
    "ck_swiglu_bwd_grouped": (
        c_int32,
        [c_void_p, c_void_p, c_int32, c_void_p, c_void_p, c_void_p, c_int32, c_int64, c_void_p, c_void_p, c_int64, c_int32, c_int32, c_void_p],
    ),
    "ck_transpose_batched": (c_int32, [c_void_p, c_int64, c_int32, c_int32, c_void_p, c_int32, c_void_p]),
    "ck_grouped_gemm": (
        c_int32,
        [c_void_p, c_int32, c_void_p, c_int32, c_int32, POINTER(ck_segments), c_int32, c_void_p, c_void_p, c_int64, c_void_p, c_void_p, c_int32, c_void_p],
    ),
    "ck_grouped_gemm_workspace_bytes": (c_int64, []),
    "ck_grouped_gemm_ws": (
        c_int32,
        [c_void_p, c_int32, c_void_p, c_int32, c_int32, POINTER(ck_segments), c_int32, c_void_p, c_void_p, c_int64, c_void_p, c_void_p, c_int32, c_void_p, c_void_p, c_int64],
    ),
    "ck_grouped_gemm_nn_ws": (
        c_int32,
        [c_void_p, c_void_p, c_int32, c_int32, POINTER(ck_segments), c_int32, c_void_p, c_int32, c_void_p, c_void_p, c_int64],
    ),
    "ck_grouped_gemm_nn": (c_int32, [c_void_p, c_void_p, c_int32, c_int32, POINTER(ck_segments), c_int32, c_void_p, c_int32, c_void_p]),
    "ck_grouped_gemm_dw": (c_int32, [c_void_p, c_void_p, c_int64, c_int32, c_int32, POINTER(ck_segments), c_void_p, c_int32, c_void_p]),
    "ck_grouped_gemm_dw_rows": (c_int32, [c_void_p, c_void_p, c_int32, c_int32, POINTER(ck_segments), c_void_p, c_int32, c_void_p]),
    "ck_quant_rows_e4m3": (c_int32, [c_void_p, c_int64, c_int32, c_void_p, c_void_p, c_int32, c_void_p]),
    "ck_grouped_gemm_fp8": (
        c_int32,
        [c_void_p, c_void_p, c_int32, c_void_p, c_void_p, c_int32, c_int32, POINTER(ck_segments), c_int32, c_void_p, c_void_p, c_int32, c_void_p],
    ),
    "ck_swiglu_fwd": (c_int32, [c_void_p, c_int64, c_void_p, c_int64, c_void_p, c_int64, c_int64, c_int64, c_int32, c_void_p]),
    "ck_rmsnorm_route": (
        c_int32,
        [c_void_p, c_void_p, c_void_p, c_float, c_int64, c_int32, c_int32, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int32, c_void_p],
    ),
    "ck_grouped_gemm_f32": (
        c_int32,
        [c_void_p, c_int32, c_void_p, c_int32, c_int32, c_int32, POINTER(ck_segments), c_int32, c_void_p, c_void_p, c_void_p],
    ),
    "ck_grouped_gemm_dw_f32": (c_int32, [c_void_p, c_void_p, c_int32, c_int32, POINTER(ck_segments), c_void_p, c_void_p]),
    "ck_gelu_tanh_bwd": (c_int32, [c_void_p, c_void_p, c_void_p, c_int64, c_int32, c_void_p]),
    "ck_swiglu_bwd": (
        c_int32,
        [c_void_p, c_int64, c_void_p, c_int64, c_void_p, c_int64, c_void_p, c_int64, c_void_p, c_int64, c_int64, c_int64, c_int32, c_void_p],
    ),
    "ck_rmsnorm_fwd": (c_int32, [c_void_p, c_void_p, c_float, c_int64, c_int32, c_void_p, c_void_p, c_int32, c_void_p]),
    "ck_rmsnorm_bwd_partial_rows": (c_int64, [c_int64]),
    "ck_rmsnorm_bwd": (c_int32, [c_void_p, c_void_p, c_void_p, c_void_p, c_float, c_int64, c_int32, c_void_p, c_void_p, c_void_p, c_int32, c_void_p]),
    "ck_add_expert_bias": (c_int32, [c_void_p, c_int64, c_int32, c_void_p, c_void_p, POINTER(ck_segments), c_int32, c_void_p]),
    "ck_expert_bias_grad": (c_int32, [c_void_p, c_int32, POINTER(ck_segments), c_void_p, c_int32, c_void_p]),
    "ck_softmax_fwd": (c_int32, [c_void_p, c_float, c_int64, c_int32, c_void_p, c_int32, c_void_p]),
    "ck_softmax_bwd": (c_int32, [c_void_p, c_void_p, c_float, c_int64, c_int32, c_void_p, c_int32, c_void_p]),
    "ck_fused_residual_add_rmsnorm_fwd": (c_int32, [c_void_p, c_void_p, c_void_p, c_float, c_float, c_int64, c_int32, c_void_p, c_void_p, c_void_p, c_int32, c_void_p]),
    "ck_fused_residual_add_rmsnorm_bwd": (c_int32, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_float, c_float, c_int64, c_int32, c_void_p, c_void_p, c_void_p, c_void_p, c_int32, c_void_p]),
}

EXPORTED_SYMBOLS = tuple(_SIGNATURES)

_lib = None


def library_path() -> str:
    return _LIB_PATH


def use_library(path: str) -> None:
    """Load another build of the library (a measurement build made with build.py --define ... --output FILE.so) instead
    of the product one. Must be called before the first kernel call of the process; bench.py --lib does. Still no
    fallback: a missing file raises on first use."""
    global _LIB_PATH
    if _lib is not None:
        raise RuntimeError("use_library: the library is already loaded")
    _LIB_PATH = os.path.abspath(path)


def set_option(name: str, value: int) -> None:
    """ck_debug_set_option: choose between kernels that compute the same result (tests and measurements)."""
    check(lib().ck_debug_set_option(name.encode(), int(value)))


def lib() -> ctypes.CDLL:
    """dlopen the library on first use; raise if it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            raise RuntimeError(
                f"{_LIB_NAME} is not built ({_LIB_PATH} is missing). Run `python cute-kernels_amd/build.py` "
                "(needs hipcc; cross-compiles for gfx950 without a GPU)."
            )
        handle = ctypes.CDLL(_LIB_PATH)
        for name, (restype, argtypes) in _SIGNATURES.items():
            fn = getattr(handle, name)  # AttributeError here = header and library disagree
            fn.restype = restype
            fn.argtypes = argtypes
        _lib = handle
    return _lib


def check(rc: int) -> None:
    if rc != 0:
        raise RuntimeError(lib().ck_last_error_string().decode())


def dtype_code(dtype: torch.dtype) -> int:
    try:
        return _DTYPE_CODES[dtype]
    except KeyError:
        raise NotImplementedError(f"libck_mi355 has no kernels for dtype {dtype}") from None


def ptr(t: torch.Tensor | None) -> int | None:
    """Device address of a tensor (None -> NULL)."""
    if t is None:
        return None
    return t.data_ptr()


def require_gpu(*tensors: torch.Tensor) -> None:
    for t in tensors:
        if t is not None and not t.is_cuda:
            raise RuntimeError(
                "cute_kernels (MI355X build) runs on the GPU only; got a tensor on " f"{t.device}. There is no CPU path."
            )


def stream() -> int:
    return torch.cuda.current_stream().cuda_stream


_zero_workspaces: dict = {}


def zero_workspace(device: torch.device, words: int, kind: str) -> torch.Tensor:
    """A uint32 workspace that starts all-zero; the kernels using it restore the words they require to be zero.

    One buffer per (kind, device, stream): calls on one stream are ordered, calls on different streams never share
    it, and kernels with different zero-invariants (kind) never share it either.
    """
    key = (kind, device.index, stream())
    buf = _zero_workspaces.get(key)
    if buf is None or buf.numel() < words:
        buf = torch.zeros(max(words, 1 << 16), dtype=torch.int32, device=device)
        _zero_workspaces[key] = buf
    return buf
