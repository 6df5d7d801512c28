"""score_mods that add custom inputs or index terms to the score (the custom-input classes of
core/lower/lower.py:561-615, ALiBi, soft-capping), through the operators AttentionEngine returns and through the C
ABI, against oracle.biased_attention.  Tolerance atol 2e-2 / rtol 1e-2."""
import math

import pytest
import torch

import oracle
from oracle import inputs
import specs
from attn_engine import AttentionEngine
from core import CustomIO

pytestmark = pytest.mark.gpu
ATOL, RTOL = 2e-2, 1e-2


def _engine(B, H, S, D, io, score_mod, causal, online=None, dtype=torch.bfloat16):
    return AttentionEngine(specs._meta(B, H, S, D, D, dtype), CustomIO(io), score_mod=score_mod,
                           mask_mod=specs.causal_mask if causal else None, online_func=online or specs.OnlineSoftmax())


@pytest.mark.parametrize("D,S,causal", [(128, 200, True), (64, 333, False)])
def test_additive_tile(D, S, causal):
    """A relative-position bias tile (1, heads, seq_len, seq_len_kv) in the tensor dtype (class b of lower.py:591-598)."""
    B, H = 2, 3
    scale = D ** -0.5
    mod = _engine(B, H, S, D, {"rel": (1, "heads", "seq_len", "seq_len_kv")},
                  lambda s, c, b, h, q, k: s * scale + c.input_tensors["rel"], causal)
    q, k, v = inputs.softmax_inputs(B, H, S, D, D, seed=S)
    rel = torch.randn(1, H, S, S, generator=torch.Generator().manual_seed(1)).bfloat16()
    o = mod(q.cuda(), k.cuda(), v.cuda(), rel.cuda())
    torch.cuda.synchronize()
    ref, lse = oracle.biased_attention(q, k, v, add=rel.float(), causal=causal, softmax_scale=scale, return_lse=True)
    oracle.assert_close(o.float().cpu(), ref, rtol=RTOL, atol=ATOL)
    torch.testing.assert_close(mod.final_rowscales.cpu(), lse, rtol=1e-4, atol=1e-4)


def test_kv_vector_and_per_row_tensor_sigmoid():
    """An fp32 seq_len_kv vector (class c, lower.py:599-603) and an fp32 (batch, heads, seq_len) tensor (class a,
    :587-590) added inside a sigmoid score function, with a one-element bias tensor beside them."""
    B, H, S, D = 2, 2, 192, 128
    io = {"colv": ("seq_len_kv",), "rowt": ("batch", "heads", "seq_len"), "b1": (1,)}

    def score_mod(s, c, b, h, q, k):
        t = c.input_tensors
        x = (s + t["colv"]) * 0.05 + t["rowt"] + t["b1"]
        return 1 / (1 + (-x).exp())

    mod = _engine(B, H, S, D, io, score_mod, True, online=specs.OnlineIdentity())
    q, k, v = inputs.softmax_inputs(B, H, S, D, D, seed=9)
    g = torch.Generator().manual_seed(2)
    colv, rowt, b1 = torch.randn(S, generator=g) * 4, torch.randn(B, H, S, generator=g), torch.tensor([-3.0])
    o = mod(q.cuda(), k.cuda(), v.cuda(), colv.cuda(), rowt.cuda(), b1.cuda())
    torch.cuda.synchronize()
    add = colv.view(1, 1, 1, S) * 0.05 + rowt.view(B, H, S, 1)
    ref = oracle.biased_attention(q, k, v, add=add, causal=True, family="sigmoid", softmax_scale=0.05, bias=-3.0)
    oracle.assert_close(o.float().cpu(), ref, rtol=RTOL, atol=ATOL, mismatch_ratio=2e-3)


@pytest.mark.parametrize("per_head", [True, False])
def test_alibi(per_head):
    """score * scale - slope[h] * (q_idx - kv_idx): slopes as a per-head custom tensor, or one constant."""
    B, H, S, D = 1, 4, 300, 128
    scale = D ** -0.5
    slopes = torch.tensor([2.0 ** -(i + 1) for i in range(H)])
    if per_head:
        mod = _engine(B, H, S, D, {"slopes": ("heads",)}, lambda s, c, b, h, q, k: s * scale - c.input_tensors["slopes"] * (q - k), True)
        extra = (slopes.cuda(),)
    else:
        slopes = torch.full((H,), 0.0625)
        mod = _engine(B, H, S, D, {}, lambda s, c, b, h, q, k: s * scale + (k - q) * 0.0625, True)
        extra = ()
    q, k, v = inputs.softmax_inputs(B, H, S, D, D, seed=12)
    o = mod(q.cuda(), k.cuda(), v.cuda(), *extra)
    torch.cuda.synchronize()
    idx = torch.arange(S, dtype=torch.float32)
    add = slopes.view(1, H, 1, 1) * (idx.view(1, 1, 1, S) - idx.view(1, 1, S, 1))
    ref = oracle.biased_attention(q, k, v, add=add, causal=True, softmax_scale=scale)
    oracle.assert_close(o.float().cpu(), ref, rtol=RTOL, atol=ATOL)


def test_softcap():
    """cap * tanh(score * scale / cap) before the softmax."""
    B, H, S, D, cap = 1, 2, 256, 128, 5.0
    scale = D ** -0.5
    mod = _engine(B, H, S, D, {}, lambda s, c, b, h, q, k: (s * (scale / cap)).tanh() * cap, True)
    q, k, v = inputs.softmax_inputs(B, H, S, D, D, seed=13)
    q = (q.float() * 3).bfloat16()          # scores well into the flat part of tanh
    o = mod(q.cuda(), k.cuda(), v.cuda())
    torch.cuda.synchronize()
    ref = oracle.biased_attention(q, k, v, causal=True, softmax_scale=scale / cap, softcap=cap)
    oracle.assert_close(o.float().cpu(), ref, rtol=RTOL, atol=ATOL)


def test_score_add_through_the_c_abi_relu_and_strides():
    """hb.attn_fwd(score_add=...) directly: a full fp32 [B, H, Sq, Skv] tensor with the relu family, and the same values
    through broadcasting views (stride 0 along batch)."""
    from metaattention_amd import hip_backend as hb
    hb.load_library()
    B, H, S, D = 2, 2, 130, 64
    q, k, v = inputs.softmax_inputs(B, H, S, D, D, seed=14)
    k, v = (k.float() * 0.5).bfloat16(), (v.float() * 0.5).bfloat16()
    add = torch.randn(1, H, S, S, generator=torch.Generator().manual_seed(3))
    ref = oracle.biased_attention(q, k, v, add=add, family="relu", softmax_scale=D ** -0.5)
    for a in (add.expand(B, H, S, S).contiguous().cuda(), add.cuda()):
        o = hb.attn_fwd(q.cuda(), k.cuda(), v.cuda(), family=hb.MA_ATTN_RELU, causal=False, scale=D ** -0.5, score_add=a)
        torch.cuda.synchronize()
        oracle.assert_close(o.float().cpu(), ref, rtol=RTOL, atol=ATOL, mismatch_ratio=2e-3)
    with pytest.raises(hb.MetaAttentionError):
        hb.attn_fwd(q.cuda(), k.cuda(), v.cuda(), family=hb.MA_ATTN_RELU, causal=False, scale=D ** -0.5, softcap=2.0)


def test_backward_through_additive_terms_is_refused():
    B, H, S, D = 1, 1, 128, 128
    mod = _engine(B, H, S, D, {"colv": ("seq_len_kv",)}, lambda s, c, b, h, q, k: s * 0.1 + c.input_tensors["colv"], True)
    q, k, v = (t.cuda().requires_grad_(True) for t in inputs.softmax_inputs(B, H, S, D, D, seed=15))
    o = mod(q, k, v, torch.zeros(S, device="cuda"))
    with pytest.raises(NotImplementedError):
        o.float().sum().backward()
