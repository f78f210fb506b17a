"""The `*_torch` names the package exports for import compatibility, checked on the CPU against the oracle."""

import os
import sys

import pytest
import torch

sys.path.insert(0, os.path.join(os.path.dirname(__file__), "..", "cute-kernels_amd"))

from oracle import moe_oracle as mo


def _ck():
    import cute_kernels

    return cute_kernels


def test_elementwise_names_match_oracle():
    ck = _ck()
    torch.manual_seed(0)
    x = torch.randn(7, 24, dtype=torch.bfloat16)
    r = torch.randn(7, 24, dtype=torch.bfloat16)
    w = torch.randn(24, dtype=torch.bfloat16)
    assert torch.equal(ck.swiglu_torch(x, r), mo.swiglu_torch(x, r))
    assert torch.equal(ck.swiglu_packed_torch(x), mo.swiglu_packed_torch(x))
    assert torch.equal(ck.rmsnorm_torch(x, w, 1e-5), mo.rmsnorm_torch(x, w, 1e-5))
    assert torch.equal(ck.rmsnorm_torch(x, None, 1e-6), mo.rmsnorm_torch(x, None, 1e-6))
    for mult in (None, 1, 0.5):
        ours, theirs = ck.fused_residual_add_rmsnorm_torch(x, r, w, 1e-5, mult), mo.fused_residual_add_rmsnorm_torch(x, r, w, 1e-5, mult)
        assert torch.equal(ours[0], theirs[0]) and torch.equal(ours[1], theirs[1])
    for mult in (None, 1, 3.0):
        assert torch.equal(ck.softmax_torch(x, mult), mo.softmax_torch(x, mult))
    ids = torch.randint(0, 9, (1000,))
    counts = ck.continuous_count_torch(ids, 9)
    assert counts.dtype == torch.uint32 and torch.equal(counts.long(), torch.bincount(ids, minlength=9))


@pytest.mark.parametrize("k,is_glu,add_bias", [(1, True, False), (2, True, True), (3, False, True)])
def test_moe_torch_matches_oracle_layer(k, is_glu, add_bias):
    ck = _ck()
    act = mo.swiglu_packed_torch if is_glu else torch.nn.GELU("tanh")
    torch.manual_seed(3)
    ours = ck.MoE_Torch(6, k, 32, 20, act, is_glu, add_bias, 0.2).double()
    theirs = mo.MoEOracle(6, k, 32, 20, act, is_glu, add_bias, 0.2).double()
    assert [(n, tuple(p.shape)) for n, p in ours.state_dict().items()] == [(n, tuple(p.shape)) for n, p in theirs.state_dict().items()]
    with torch.no_grad():
        for p in ours.parameters():
            p.normal_(0, 0.2)
    theirs.load_state_dict(ours.state_dict())
    x = torch.randn(2, 11, 32, dtype=torch.float64, requires_grad=True)
    x2 = x.detach().clone().requires_grad_()
    y, logits = ours(x)
    y2, logits2 = theirs(x2)
    assert torch.equal(logits, logits2)
    torch.testing.assert_close(y, y2, rtol=1e-12, atol=1e-12)
    g = torch.randn_like(y)
    y.backward(g)
    y2.backward(g)
    torch.testing.assert_close(x.grad, x2.grad, rtol=1e-10, atol=1e-12)
    for (n, p), (_, q) in zip(ours.named_parameters(), theirs.named_parameters()):
        torch.testing.assert_close(p.grad, q.grad, rtol=1e-10, atol=1e-12, msg=n)
