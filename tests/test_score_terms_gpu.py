"""score_mods that add custom inputs or index terms to the score (the custom-input classes of
core/lower/lower.py:561-615, ALiBi, soft-capping), through the operators AttentionEngine returns and through the C
ABI, against oracle.biased_attention, forward and (softmax family) backward.  Tolerance atol 2e-2 / rtol 1e-2, for the
gradients with the 1e-3 allowance for the rounding of p and ds that the other backward tests use."""
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


def test_scaled_and_several_one_element_tensors():
    """One-element tensors inside the scaling, `(s + t1) * scale - t2`: the kernels' bias pointer carries a lone tensor with
    coefficient 1 (examples/sigmoid_attn.py:17-21); anything else goes the way of the other additive terms.  Forward and
    backward through the operator."""
    B, H, S, D = 2, 2, 160, 128
    scale = D ** -0.5
    io = {"t1": (1,), "t2": (1,)}
    # (under softmax a constant shift cancels: the sigmoid score function keeps it visible)
    def score_mod(s, c, b, h, q, k):
        x = (s + c.input_tensors["t1"]) * scale - c.input_tensors["t2"]
        return 1 / (1 + (-x).exp())
    mod = _engine(B, H, S, D, io, score_mod, True, online=specs.OnlineIdentity())
    assert mod.score_form.bias_tensor is None and mod.score_form.extra == {("t:t1",): scale, ("t:t2",): -1.0}
    q, k, v = inputs.softmax_inputs(B, H, S, D, D, seed=12)
    t1, t2 = torch.tensor([7.0]), torch.tensor([2.5])
    qc, kc, vc = (t.cuda().requires_grad_() for t in (q, k, v))
    o = mod(qc, kc, vc, t1.cuda(), t2.cuda())
    dout = (0.5 * torch.randn(B, S, H, D, generator=torch.Generator().manual_seed(3))).bfloat16()
    o.backward(dout.cuda())
    torch.cuda.synchronize()
    kw = dict(causal=True, family="sigmoid", softmax_scale=scale, bias=7.0 * scale - 2.5)
    oracle.assert_close(o.float().cpu(), oracle.biased_attention(q, k, v, **kw), rtol=RTOL, atol=ATOL, mismatch_ratio=2e-3)
    ref = oracle.attention_grads(oracle.biased_attention, q, k, v, dout, **kw)
    for name, a, b_ in zip(("dq", "dk", "dv"), (qc.grad, kc.grad, vc.grad), ref):
        oracle.assert_close(a.float().cpu(), b_.float(), rtol=RTOL, atol=ATOL, mismatch_ratio=5e-3, msg=name)


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


def _check_grads(got, ref, what):
    for name, a, b in zip(("dq", "dk", "dv"), got, ref):
        oracle.assert_close(a.float().cpu(), b.float(), rtol=RTOL, atol=ATOL, mismatch_ratio=1e-3, msg=f"{what}:{name}")


def _engine_grads(mod, q, k, v, dout, *custom):
    qc, kc, vc = (t.cuda().requires_grad_(True) for t in (q, k, v))
    o = mod(qc, kc, vc, *custom)
    o.backward(dout.cuda())
    torch.cuda.synchronize()
    return o, (qc.grad, kc.grad, vc.grad)


@pytest.mark.parametrize("D,S,causal", [(128, 200, True), (64, 333, False)])
def test_backward_through_an_additive_tile(D, S, causal):
    """Gradients of q, k, v through score * scale + rel[h, q, kv] (the custom input itself gets none, as in the
    reference, attn_tl.py:692), against autograd over oracle.biased_attention in fp64."""
    B, H = 2, 3
    scale = D ** -0.5
    mod = _engine(B, H, S, D, {"rel": (1, "heads", "seq_len", "seq_len_kv")},
                  lambda s, c, b, h, q, k: s * scale + c.input_tensors["rel"], causal)
    q, k, v = inputs.softmax_inputs(B, H, S, D, D, seed=S)
    g = torch.Generator().manual_seed(4)
    rel = torch.randn(1, H, S, S, generator=g).bfloat16()
    dout = torch.randn(B, S, H, D, generator=g).bfloat16()
    rel_c = rel.cuda().requires_grad_(True)
    print(f"bwd additive tile D{D} S{S} causal={causal}", flush=True)
    o, got = _engine_grads(mod, q, k, v, dout, rel_c)
    assert rel_c.grad is None
    oracle.assert_close(o.float().cpu(), oracle.biased_attention(q, k, v, add=rel.float(), causal=causal, softmax_scale=scale),
                        rtol=RTOL, atol=ATOL)
    ref = oracle.attention_grads(oracle.biased_attention, q, k, v, dout, add=rel.double(), causal=causal, softmax_scale=scale)
    _check_grads(got, ref, "additive tile")
    # the term matters: without it the gradients are different ones
    plain = oracle.attention_grads(oracle.biased_attention, q, k, v, dout, causal=causal, softmax_scale=scale)
    assert not torch.allclose(got[0].float().cpu(), plain[0].float(), rtol=1e-1, atol=1e-1)


def test_backward_through_an_additive_tile_under_a_sliding_window():
    """A mask_mod that is neither causal nor absent (the element-mask path of the backward kernels) together with an
    additive tile; the oracle takes the window as -inf entries of the added term."""
    B, H, S, D = 1, 2, 384, 128
    scale = D ** -0.5
    window = lambda b, h, q, k: (q >= k) & (q - k < 100)
    mod = AttentionEngine(specs._meta(B, H, S, D, D, torch.bfloat16), CustomIO({"rel": (1, "heads", "seq_len", "seq_len_kv")}),
                          score_mod=lambda s, c, b, h, q, k: s * scale + c.input_tensors["rel"], mask_mod=window,
                          online_func=specs.OnlineSoftmax())
    q, k, v = inputs.softmax_inputs(B, H, S, D, D, seed=17)
    g = torch.Generator().manual_seed(7)
    rel = torch.randn(1, H, S, S, generator=g)
    dout = torch.randn(B, S, H, D, generator=g).bfloat16()
    print("bwd additive tile + sliding window", flush=True)
    o, got = _engine_grads(mod, q, k, v, dout, rel.cuda())
    idx = torch.arange(S)
    keep = window(0, 0, idx.view(S, 1), idx.view(1, S))
    add = rel.double().masked_fill(~keep, float("-inf"))
    oracle.assert_close(o.float().cpu(), oracle.biased_attention(q, k, v, add=add.float(), softmax_scale=scale), rtol=RTOL, atol=ATOL)
    ref = oracle.attention_grads(oracle.biased_attention, q, k, v, dout, add=add, softmax_scale=scale)
    _check_grads(got, ref, "window + tile")


def test_backward_through_alibi_and_a_kv_vector():
    """Per-head slopes on both indices and an fp32 seq_len_kv vector in one score_mod."""
    B, H, S, D = 1, 4, 300, 128
    scale = D ** -0.5
    slopes = torch.tensor([2.0 ** -(i + 1) for i in range(H)])
    mod = _engine(B, H, S, D, {"slopes": ("heads",), "colv": ("seq_len_kv",)},
                  lambda s, c, b, h, q, k: s * scale - c.input_tensors["slopes"] * (q - k) + c.input_tensors["colv"], True)
    q, k, v = inputs.softmax_inputs(B, H, S, D, D, seed=16)
    g = torch.Generator().manual_seed(5)
    colv = torch.randn(S, generator=g) * 2
    dout = torch.randn(B, S, H, D, generator=g).bfloat16()
    print("bwd alibi + kv vector", flush=True)
    _, got = _engine_grads(mod, q, k, v, dout, slopes.cuda(), colv.cuda())
    idx = torch.arange(S, dtype=torch.float64)
    add = slopes.double().view(1, H, 1, 1) * (idx.view(1, 1, 1, S) - idx.view(1, 1, S, 1)) + colv.double().view(1, 1, 1, S)
    ref = oracle.attention_grads(oracle.biased_attention, q, k, v, dout, add=add, causal=True, softmax_scale=scale)
    _check_grads(got, ref, "alibi")


def test_backward_through_softcap():
    """cap * tanh(score * scale / cap): ds carries the factor cap * (1 - tanh^2) * scale / cap."""
    B, H, S, D, cap = 1, 2, 256, 128, 5.0
    scale = D ** -0.5
    mod = _engine(B, H, S, D, {}, lambda s, c, b, h, q, k: (s * (scale / cap)).tanh() * cap, True)
    q, k, v = inputs.softmax_inputs(B, H, S, D, D, seed=13)
    q = (q.float() * 3).bfloat16()          # scores well into the flat part of tanh
    dout = torch.randn(B, S, H, D, generator=torch.Generator().manual_seed(6)).bfloat16()
    print("bwd softcap", flush=True)
    _, got = _engine_grads(mod, q, k, v, dout)
    ref = oracle.attention_grads(oracle.biased_attention, q, k, v, dout, causal=True, softmax_scale=scale / cap, softcap=cap)
    _check_grads(got, ref, "softcap")
    plain = oracle.attention_grads(oracle.biased_attention, q, k, v, dout, causal=True, softmax_scale=scale)
    assert not torch.allclose(got[0].float().cpu(), plain[0].float(), rtol=1e-1, atol=1e-1)


@pytest.mark.parametrize("D,DV,H,Hkv,Sq,Skv,causal,dtype", [(128, 128, 4, 2, 200, 200, True, torch.bfloat16),
                                                           (64, 64, 2, 2, 70, 333, False, torch.float16),
                                                           (256, 512, 2, 1, 160, 160, True, torch.bfloat16),
                                                           (128, 256, 2, 2, 1100, 1100, True, torch.bfloat16),
                                                           (192, 128, 2, 1, 300, 300, True, torch.float16)])
def test_attn_bwd_score_terms_through_the_c_abi(D, DV, H, Hkv, Sq, Skv, causal, dtype):
    """hb.attn_bwd(score_add=..., pos_slope_*=..., softcap=...) directly: every head-size pair of the backward kernels,
    grouped kv heads, unequal lengths, an fp32 tile broadcast over batch (stride 0), all terms at once."""
    from metaattention_amd import hip_backend as hb
    hb.load_library()
    B, scale, cap = 2, D ** -0.5, 4.0
    g = torch.Generator().manual_seed(Sq + D)
    q = torch.randn(B, Sq, H, D, generator=g).to(dtype)
    k = torch.randn(B, Skv, Hkv, D, generator=g).to(dtype)
    v = torch.randn(B, Skv, Hkv, DV, generator=g).to(dtype)
    dout = torch.randn(B, Sq, H, DV, generator=g).to(dtype)
    add = torch.randn(1, H, Sq, Skv, generator=g)
    sq, sk = torch.rand(H, generator=g) * 0.01, -torch.rand(H, generator=g) * 0.01
    kw = dict(family=hb.MA_ATTN_SOFTMAX, causal=causal, scale=scale, bias=0.1, score_add=add.cuda(), pos_slope_q=sq.cuda(),
              pos_slope_kv=sk.cuda(), softcap=cap)
    print(f"attn_bwd score terms D{D} DV{DV} H{H}/{Hkv} S{Sq}x{Skv} causal={causal} {dtype}", flush=True)
    qc, kc, vc = q.cuda(), k.cuda(), v.cuda()
    lse = torch.empty(B, H, Sq, device="cuda")
    o = hb.attn_fwd(qc, kc, vc, row_scale=lse, **kw)
    got = hb.attn_bwd(qc, kc, vc, o, dout.cuda(), lse, **kw)
    torch.cuda.synchronize()
    iq, ik = torch.arange(Sq, dtype=torch.float64), torch.arange(Skv, dtype=torch.float64)
    full = add.double() + sq.double().view(1, H, 1, 1) * iq.view(1, 1, Sq, 1) + sk.double().view(1, H, 1, 1) * ik.view(1, 1, 1, Skv)
    oracle.assert_close(o.float().cpu(), oracle.biased_attention(q, k, v, add=full.float(), causal=causal, softmax_scale=scale, bias=0.1,
                                                                 softcap=cap), rtol=RTOL, atol=ATOL)
    ref = oracle.attention_grads(oracle.biased_attention, q, k, v, dout, add=full, causal=causal, softmax_scale=scale, bias=0.1, softcap=cap)
    _check_grads(got, ref, "c abi")


def test_backward_through_additive_terms_sigmoid_and_relu():
    """The sigmoid and relu families differentiate through additive terms as well (the score function sees x = s * scale +
    bias + added terms): an fp32 key vector and a per-row tensor inside a sigmoid spec through the engine, a tile with
    relu through the C ABI."""
    from metaattention_amd import hip_backend as hb
    hb.load_library()
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
    dout = (0.25 * torch.randn(B, S, H, D, generator=g)).bfloat16()
    print("bwd sigmoid with additive terms", flush=True)
    _, got = _engine_grads(mod, q, k, v, dout, colv.cuda(), rowt.cuda(), b1.cuda())
    add = colv.double().view(1, 1, 1, S) * 0.05 + rowt.double().view(B, H, S, 1)
    ref = oracle.attention_grads(oracle.biased_attention, q, k, v, dout, add=add, causal=True, family="sigmoid", softmax_scale=0.05, bias=-3.0)
    _check_grads(got, ref, "sigmoid + terms")

    D2, S2 = 64, 130
    q, k, v = inputs.softmax_inputs(B, H, S2, D2, D2, seed=14)
    k, v = (k.float() * 0.5).bfloat16(), (v.float() * 0.5).bfloat16()
    add = torch.randn(1, H, S2, S2, generator=g)
    dout = (0.25 * torch.randn(B, S2, H, D2, generator=g)).bfloat16()
    kw = dict(family=hb.MA_ATTN_RELU, causal=False, scale=D2 ** -0.5, score_add=add.cuda())
    print("bwd relu with an additive tile", flush=True)
    o = hb.attn_fwd(q.cuda(), k.cuda(), v.cuda(), **kw)
    got = hb.attn_bwd(q.cuda(), k.cuda(), v.cuda(), o, dout.cuda(), None, **kw)
    torch.cuda.synchronize()
    ref = oracle.attention_grads(oracle.biased_attention, q, k, v, dout, add=add.double(), family="relu", softmax_scale=D2 ** -0.5)
    for name, a, b in zip(("dq", "dk", "dv"), got, ref):
        oracle.assert_close(a.float().cpu(), b.float(), rtol=RTOL, atol=ATOL, mismatch_ratio=2e-3, msg=f"relu + tile:{name}")


def test_soft_capping_outside_the_softmax_family_is_refused():
    """cap * tanh(x) goes with the softmax row function only, forward and backward: loud, not silently wrong."""
    from metaattention_amd import hip_backend as hb
    hb.load_library()
    B, H, S, D = 1, 1, 128, 128
    q, k, v = (t.cuda() for t in inputs.softmax_inputs(B, H, S, D, D, seed=15))
    with pytest.raises(hb.MetaAttentionError):
        hb.attn_bwd(q, k, v, q, q, None, family=hb.MA_ATTN_SIGMOID, causal=True, scale=0.1, softcap=2.0)
    lse = torch.zeros(B, H, S, device="cuda")
    mask = torch.ones(1, H, S, S, device="cuda", dtype=torch.bfloat16)
    with pytest.raises(hb.MetaAttentionError):
        hb.attn_bwd(q, k, v, q, q, lse, family=hb.MA_ATTN_RETENTION, causal=True, scale=1.0, score_mask=mask, score_mask_t=mask,
                    score_add=torch.zeros(1, 1, S, S, device="cuda"))
