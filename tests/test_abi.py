"""CPU-side checks of the drop-in boundary: the C-ABI library loads, exports every symbol include/ck_mi355.h declares,
rejects bad arguments with a message (no GPU needed: validation precedes any launch), and the Python API surface has the
reference's names, signatures and error behaviour."""

import inspect
import os
import re

import pytest
import torch

import cute_kernels
from cute_kernels import _C

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "ck_mi355.h")


def _declared_symbols() -> set[str]:
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return set(re.findall(r"\b(ck_[a-z0-9_]+)\s*\(", text))


def test_library_exports_every_declared_symbol():
    declared = _declared_symbols()
    assert len(declared) >= 20
    lib = _C.lib()
    for name in declared:
        assert hasattr(lib, name), f"{name} is declared in ck_mi355.h but not exported"
    assert declared == set(_C.EXPORTED_SYMBOLS), "ctypes signature table and header disagree"
    assert lib.ck_abi_version() == 2


def test_argument_validation_returns_error_and_message():
    lib = _C.lib()
    assert lib.ck_count_offsets(None, 0, 10, 0, None, None, None, None, None) != 0
    assert b"num_bins" in lib.ck_last_error_string()
    assert lib.ck_count_offsets(None, 0, 10, 20000, None, None, None, None, None) != 0
    assert lib.ck_route_topk_softmax(None, _C.CK_BF16, 4, 8, 9, None, None, None, None) != 0
    assert b"k=9" in lib.ck_last_error_string()
    assert lib.ck_route_topk_softmax(None, 7, 4, 8, 2, 1, 1, None, None) != 0  # unknown dtype code
    assert lib.ck_swiglu_fwd(None, 0, None, 0, None, 0, -1, 4, _C.CK_F32, None) != 0
    assert lib.ck_rmsnorm_fwd(None, None, 1e-6, 4, 0, None, None, _C.CK_F32, None) != 0
    with pytest.raises(RuntimeError, match="H=0"):
        _C.check(lib.ck_rmsnorm_fwd(None, None, 1e-6, 4, 0, None, None, _C.CK_F32, None))


def test_host_side_size_helpers():
    lib = _C.lib()
    assert lib.ck_count_workspace_words(64) == 1 + 64 * 32
    assert lib.ck_count_workspace_words(16384) == 1 + 16384
    # sum_e round_up(c_e, align) <= R + E*(align-1), rounded to whole tiles
    assert lib.ck_sort_max_rows(32768, 8, 256) == 34816
    assert lib.ck_sort_max_rows(0, 8, 128) % 128 == 0
    for R, E, align in [(1, 128, 128), (65536, 64, 128), (524288, 128, 256)]:
        m = lib.ck_sort_max_rows(R, E, align)
        assert m % align == 0 and m >= R + E * (align - 1)
    assert lib.ck_sort_workspace_words(32768, 8) >= 1 + 8
    assert lib.ck_rmsnorm_bwd_partial_rows(0) == 0
    assert lib.ck_rmsnorm_bwd_partial_rows(10**6) == 2048


def test_python_api_surface_matches_reference_names_and_signatures():
    for name in ["MoE", "MoE_Triton", "continuous_count_cute", "swiglu_cute", "swiglu_packed_cute", "rmsnorm_cute",
                 "set_seed", "ceil_divide"]:
        assert hasattr(cute_kernels, name)
    from cute_kernels.modules import MoE  # north star's stated location

    assert list(inspect.signature(MoE.__init__).parameters)[1:] == [
        "num_experts", "num_experts_per_tok", "hidden_size", "intermediate_size", "activation_function", "is_glu",
        "add_bias", "std",
    ]
    assert list(inspect.signature(cute_kernels.continuous_count_cute).parameters) == ["x", "size"]
    sig = inspect.signature(cute_kernels.swiglu_cute)
    assert list(sig.parameters) == ["gate", "up", "kernel_backend_forward", "kernel_backend_backward"]
    assert sig.parameters["kernel_backend_forward"].kind is inspect.Parameter.KEYWORD_ONLY
    # the selector enum of the reference (kernel_backend.py:11-13) exists so that such calls still read
    assert {m.name for m in cute_kernels.KernelBackend} == {"cuda", "triton"}
    sig = inspect.signature(cute_kernels.rmsnorm_cute)
    assert list(sig.parameters) == ["x", "weight", "eps", "memory_efficient"]
    assert sig.parameters["memory_efficient"].default is False
    for m in ["_compute_routing_weights", "_compute_experts", "_get_topk"]:
        assert hasattr(MoE, m)


def test_module_state_dict_contract_and_init():
    moe = cute_kernels.MoE(4, 2, 16, 24, cute_kernels.swiglu_packed_cute, True, False, 0.02)
    sd = moe.state_dict()
    assert list(sd) == ["gate.weight", "c_fc.weight", "c_proj.weight"]
    assert sd["c_fc.weight"].shape == (4, 48, 16) and sd["c_proj.weight"].shape == (4, 16, 24)
    assert moe.top_k == 2 and moe.num_experts == 4 and moe.hidden_size == 16 and moe.intermediate_size == 24
    biased = cute_kernels.MoE(4, 2, 16, 24, cute_kernels.swiglu_packed_cute, True, True, 0.02)
    assert list(biased.state_dict()) == ["gate.weight", "c_fc.weight", "c_fc.bias", "c_proj.weight", "c_proj.bias"]
    assert float(biased.c_fc.bias.detach().abs().sum()) == 0.0
    # state dicts interchange with the oracle restatement of the reference module
    from oracle.moe_oracle import MoEOracle, swiglu_packed_torch

    MoEOracle(4, 2, 16, 24, swiglu_packed_torch, True, False, 0.02).load_state_dict(sd)


def test_no_cpu_fallback_and_reference_asserts():
    # the size == 1 shortcut comes before every check, as in the reference (continuous_count/__init__.py:26-27)
    out = cute_kernels.continuous_count_cute(torch.zeros(3, 5), 1)
    assert out.dtype == torch.uint32 and out.tolist() == [15]
    with pytest.raises(AssertionError, match="1-dimensional"):
        cute_kernels.continuous_count_cute(torch.zeros(3, 5, dtype=torch.int32), 4)
    with pytest.raises(AssertionError):
        cute_kernels.continuous_count_cute(torch.zeros(3), 4)
    with pytest.raises(RuntimeError, match="no CPU path"):
        cute_kernels.continuous_count_cute(torch.zeros(3, dtype=torch.int32), 4)
    with pytest.raises(AssertionError, match="same shape"):
        cute_kernels.swiglu_cute(torch.zeros(3), torch.zeros(4))
    with pytest.raises(RuntimeError, match="no CPU path"):
        cute_kernels.swiglu_cute(torch.zeros(4), torch.zeros(4))
    with pytest.raises(AssertionError, match="weight should be 1D"):
        cute_kernels.rmsnorm_cute(torch.zeros(2, 4), torch.zeros(2, 4), 1e-5)
    with pytest.raises(RuntimeError, match="no CPU path"):
        cute_kernels.rmsnorm_cute(torch.zeros(2, 4), None, 1e-5)
    moe = cute_kernels.MoE(4, 2, 16, 24, cute_kernels.swiglu_packed_cute, True, False, 0.02)
    with pytest.raises(RuntimeError, match="no CPU path"):
        moe(torch.zeros(3, 16))


def test_missing_library_fails_loudly(monkeypatch):
    monkeypatch.setattr(_C, "_lib", None)
    monkeypatch.setattr(_C, "_LIB_PATH", "/nonexistent/libck_mi355.so")
    with pytest.raises(RuntimeError, match="not built"):
        _C.lib()
