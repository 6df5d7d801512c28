"""The operators AttentionEngine returns for user specs, called with the
reference's layouts and argument order, against the CPU oracle."""
import math

import pytest
import torch

import oracle
from oracle import inputs
import specs

pytestmark = pytest.mark.gpu
ATOL, RTOL = 2e-2, 1e-2


@pytest.mark.parametrize("online", ["plain", "respelled"])
def test_softmax_operator(online):
    B, H, S, D = 1, 4, 512, 128
    mod = specs.softmax_attention(B, H, S, D, D, online=specs.OnlineSoftmaxRespelled() if online == "respelled" else None)
    q, k, v = inputs.softmax_inputs(B, H, S, D, D, seed=1)
    o = mod(q.cuda(), k.cuda(), v.cuda())
    torch.cuda.synchronize()
    assert o.shape == (B, S, H, D) and o.dtype == torch.bfloat16
    ref, lse = oracle.softmax_attention(q, k, v, causal=True, return_lse=True)
    oracle.assert_close(o.float().cpu(), ref, rtol=RTOL, atol=ATOL)
    torch.testing.assert_close(mod.final_rowscales.cpu(), lse, rtol=1e-4, atol=1e-4)


def test_softmax_operator_fp16_noncausal():
    B, H, S, D = 2, 2, 256, 128
    mod = specs.softmax_attention(B, H, S, D, D, dtype=torch.float16, causal=False)
    q, k, v = inputs.softmax_inputs(B, H, S, D, D, dtype=torch.float16, seed=2)
    o = mod(q.cuda(), k.cuda(), v.cuda())
    torch.cuda.synchronize()
    oracle.assert_close(o.float().cpu(), oracle.softmax_attention(q, k, v, causal=False), rtol=RTOL, atol=ATOL)


def test_sigmoid_operator_with_bias_tensor():
    """mod(q, k, v, softmax_bias[1]) as in testing/test.py:552-566."""
    B, H, S, D = 1, 2, 256, 128
    mod = specs.sigmoid_attention(B, H, S, D, D)
    q, k, v = inputs.softmax_inputs(B, H, S, D, D, seed=3)
    q = (q.float() * 0.3).bfloat16()
    bias = torch.tensor([-4.25])
    o = mod(q.cuda(), k.cuda(), v.cuda(), bias.cuda())
    torch.cuda.synchronize()
    oracle.assert_close(o.float().cpu(), oracle.sigmoid_attention(q, k, v, bias, causal=True), rtol=RTOL, atol=ATOL, mismatch_ratio=2e-3)


def test_sigmoid_operator_scaled_constant_bias():
    """The benchmark's variant: sigmoid(q.k * scale - log S), written with exp()."""
    B, H, S, D = 1, 2, 512, 128
    mod = specs.sigmoid_attention(B, H, S, D, D, scale=D ** -0.5, const_bias=-math.log(S), form="exp")
    q, k, v = inputs.softmax_inputs(B, H, S, D, D, seed=4)
    o = mod(q.cuda(), k.cuda(), v.cuda())
    torch.cuda.synchronize()
    ref = oracle.sigmoid_attention(q, k, v, -math.log(S), causal=True, softmax_scale=D ** -0.5)
    oracle.assert_close(o.float().cpu(), ref, rtol=RTOL, atol=ATOL)


def test_outputs_carry_a_grad_fn_and_backward_runs():
    """The operator is a torch.autograd.Function.apply (attn_tl.py:694): outputs carry grad_fn, backward fills
    q.grad / k.grad / v.grad (values are checked in test_attn_bwd_gpu.py)."""
    B, H, S, D = 1, 1, 128, 128
    mod = specs.softmax_attention(B, H, S, D, D)
    q, k, v = (t.cuda().requires_grad_(True) for t in inputs.softmax_inputs(B, H, S, D, D, seed=5))
    o = mod(q, k, v)
    assert o.grad_fn is not None
    o.float().sum().backward()
    torch.cuda.synchronize()
    for t in (q, k, v):
        assert t.grad is not None and t.grad.shape == t.shape and torch.isfinite(t.grad.float()).all()


def test_wrong_custom_tensor_count():
    mod = specs.sigmoid_attention(1, 1, 128, 128, 128)
    q = torch.zeros(1, 128, 1, 128, device="cuda", dtype=torch.bfloat16)
    with pytest.raises(TypeError):
        mod(q, q, q)
