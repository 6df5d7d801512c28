"""Host-side logic (no GPU): tracing, canonicalisation, mask helpers, and the
spec interpreter checked against the oracle (this is also how the fp32
B=1 H=4 S=512 D=64 non-causal configuration runs: on the CPU, through the traced spec)."""
import math

import pytest
import torch

import oracle
from oracle import inputs
import specs
from attn_engine import AttentionEngine, OnlineFunc
from core import CustomIO, SymbolScalar, SymbolicArray, Var, meta_tensor
from core.canonical import canonicalize_score_mod, identify_online_func, classify_mask
from core.eager import attention_by_spec
from core.transform.core import create_block_mask, is_causal_mask, is_less_causal_mask, create_mask
from autotuner.arch import get_attn_device


def test_trace_structure():
    s = SymbolicArray("scores", Var("scores"))
    m = SymbolScalar("m", Var("-inf"))
    mx = s.get_reduce("max")
    assert mx.shape_idx == ["block_M"] and mx.code.type == "ReduceMax"
    m_new = m.max(mx)
    p = (s - m_new).exp()
    assert p.code.type == "Exp" and p.prev[0].code.type == "Sub" and p.shape_idx == ["block_M", "block_N"]
    assert isinstance(p, SymbolicArray) and p.get_reduce("abssum").code.type == "ReduceAbsSum"
    c = (s * 2 + 1) / 3
    assert [c.code.type, c.prev[0].code.type, c.prev[0].prev[0].code.type] == ["Div", "Add", "Mul"]
    assert c.prev[1].code.type == "Const" and c.prev[1].code.value == 3
    assert (1 / s).code.type == "Div" and (1 - s).prev[0].code.type == "Const"
    with pytest.raises(TypeError):
        s + "x"


def test_block_mask_helpers_match_brute_force():
    # cases of attention_engine/tests/test_blockmask.py:3-26 (128x64 blocks, S=512)
    cases = {"causal": (lambda b, h, q, k: q >= k, True, True),
             "q+1>=kv": (lambda b, h, q, k: q + 1 >= k, False, False),
             "q-128>=kv": (lambda b, h, q, k: q - 128 >= k, False, True)}
    for name, (fn, exp_causal, exp_less) in cases.items():
        bm = create_block_mask(fn, 2, 4, 512, 512, "cpu", 128, 64)
        assert bm.shape == (2, 4, 4, 8) and bm.dtype == torch.int8
        dense = create_mask(fn, 2, 4, 512, 512, "cpu")
        for i in range(4):
            for j in range(8):
                assert bool(bm[0, 0, i, j]) == bool(dense[0, 0, i * 128:(i + 1) * 128, j * 64:(j + 1) * 64].any())
        assert bool(is_causal_mask(bm, 128, 64)) == exp_causal, name
        assert bool(is_less_causal_mask(bm, 128, 64)) == exp_less, name
    # ragged sizes are padded
    assert create_block_mask(lambda b, h, q, k: q >= k, 1, 1, 200, 130, "cpu", 128, 64).shape == (1, 1, 2, 3)


def test_classify_mask():
    assert classify_mask(None, 1, 2, 64, 64) == "none"
    assert classify_mask(lambda b, h, q, k: q >= k, 2, 4, 300, 300) == "causal"
    assert classify_mask(lambda b, h, q, k: (q >= k) | (q < k), 2, 4, 64, 64) == "none"
    assert classify_mask(lambda b, h, q, k: q - 4 >= k, 1, 1, 64, 64) == "other"              # shifted: element-wise keep mask
    assert classify_mask(lambda b, h, q, k: (q >= k) & (q - k < 16), 2, 4, 64, 64) == "other"  # sliding window
    assert classify_mask(lambda b, h, q, k: (q >= k) & (h > 0), 1, 2, 64, 64) == "other_bh"    # depends on the head
    assert classify_mask(lambda b, h, q, k: q >= k, 1, 1, 64, 128) == "other"                  # "causal" needs equal lengths
    # a mask that is special for one head or one batch entry only, neither the first, the middle nor the last one
    assert classify_mask(lambda b, h, q, k: (q >= k) & ((h != 1) | (k > 3)), 2, 8, 64, 64) == "other_bh"
    assert classify_mask(lambda b, h, q, k: (q >= k) | (b == 1), 5, 2, 64, 64) == "other_bh"
    doc = torch.tensor([[0] * 32 + [1] * 32, [0] * 20 + [1] * 44, [0] * 32 + [1] * 32])   # per-batch document ids, first == last
    assert classify_mask(lambda b, h, q, k: doc[b, q] == doc[b, k], 3, 2, 64, 64) == "other_bh"
    # reads b and h but does not depend on them: found by comparing every (batch, head)
    assert classify_mask(lambda b, h, q, k: (q >= k) & (b >= 0) & (h * 0 == 0), 3, 5, 64, 64) == "causal"
    # too large to compare: counts as depending on (batch, head)
    import core.canonical as cn
    lim, cn._MASK_COMPARE_LIMIT = cn._MASK_COMPARE_LIMIT, 1000
    try:
        assert classify_mask(lambda b, h, q, k: (q >= k) & (b >= 0), 3, 5, 64, 64) == "other_bh"
        assert classify_mask(lambda b, h, q, k: q >= k, 3, 5, 64, 64) == "causal"   # never touches b, h: one evaluation decides
    finally:
        cn._MASK_COMPARE_LIMIT = lim


def test_canonical_score_forms():
    io = CustomIO({"softmax_bias": (1,), "mask": (1, "heads", "seq_len", "seq_len_kv")})
    t = io.input_tensors
    f = canonicalize_score_mod(lambda s, c, b, h, q, k: s * 0.125, io)
    assert (f.activation, f.scale, f.bias, f.bias_tensor, f.mask_tensor) == ("identity", 0.125, 0.0, None, None)
    f = canonicalize_score_mod(lambda s, c, b, h, q, k: (((s + t["softmax_bias"]) * 0.5).tanh() + 1) * 0.5, io)
    assert (f.activation, f.scale, f.bias, f.bias_tensor) == ("sigmoid", 1.0, 0.0, "softmax_bias")
    f = canonicalize_score_mod(lambda s, c, b, h, q, k: 1 / (1 + (-(s * 0.25 - 3.0)).exp()), io)
    assert f.activation == "sigmoid" and abs(f.scale - 0.25) < 1e-12 and abs(f.bias + 3.0) < 1e-12
    f = canonicalize_score_mod(lambda s, c, b, h, q, k: (s / 8).max(0), io)
    assert (f.activation, f.scale) == ("relu", 0.125)
    f = canonicalize_score_mod(lambda s, c, b, h, q, k: s * t["mask"], io)
    assert (f.activation, f.scale, f.mask_tensor) == ("identity", 1.0, "mask")
    f = canonicalize_score_mod(lambda s, c, b, h, q, k: t["mask"] * (s * 0.5), io)
    assert (f.scale, f.mask_tensor) == (0.5, "mask")
    for bad in (lambda s, c, b, h, q, k: s * s, lambda s, c, b, h, q, k: s + h, lambda s, c, b, h, q, k: s.tanh() * 2 + 1,
                lambda s, c, b, h, q, k: s + q * k, lambda s, c, b, h, q, k: s.abs(), lambda s, c, b, h, q, k: s * t["mask"] + t["mask"]):
        with pytest.raises(NotImplementedError):
            canonicalize_score_mod(bad, io)


def test_canonical_additive_score_terms():
    """The custom-input classes of core/lower/lower.py:561-615 as additive terms, index terms (ALiBi), soft-capping."""
    io = CustomIO({"rel": (1, "heads", "seq_len", "seq_len_kv"), "colv": ("seq_len_kv",), "rowt": ("batch", "heads", "seq_len"),
                   "slopes": ("heads",), "b1": (1,)})
    t = io.input_tensors
    f = canonicalize_score_mod(lambda s, c, b, h, q, k: s * 0.125 + t["rel"], io)
    assert (f.activation, f.scale, f.mask_tensor, f.extra) == ("identity", 0.125, None, {("t:rel",): 1.0})
    f = canonicalize_score_mod(lambda s, c, b, h, q, k: (s + t["colv"]) * 0.125 + t["rowt"] + t["b1"], io)
    assert f.bias_tensor == "b1" and f.extra == {("t:colv",): 0.125, ("t:rowt",): 1.0}
    f = canonicalize_score_mod(lambda s, c, b, h, q, k: s * 0.125 - t["slopes"] * (q - k), io)
    assert f.extra == {("i:q_idx", "t:slopes"): -1.0, ("i:kv_idx", "t:slopes"): 1.0}
    f = canonicalize_score_mod(lambda s, c, b, h, q, k: s * 0.125 + (k - q) * 0.5, io)
    assert f.extra == {("i:kv_idx",): 0.5, ("i:q_idx",): -0.5}
    f = canonicalize_score_mod(lambda s, c, b, h, q, k: (s * (0.125 / 30)).tanh() * 30, io)
    assert f.activation == "identity" and f.softcap == 30.0 and abs(f.scale - 0.125 / 30) < 1e-12
    f = canonicalize_score_mod(lambda s, c, b, h, q, k: ((s * 0.1 + t["rel"]) * 0.5).tanh() * 0.5 + 0.5, io)
    assert f.activation == "sigmoid" and f.extra == {("t:rel",): 1.0} and abs(f.scale - 0.1) < 1e-12
    for bad in (lambda s, c, b, h, q, k: s + t["rel"] * t["colv"], lambda s, c, b, h, q, k: s + t["rowt"] * q,
                lambda s, c, b, h, q, k: s * t["rel"] + t["colv"]):
        with pytest.raises(NotImplementedError):
            canonicalize_score_mod(bad, io)


def test_identify_online_funcs():
    assert identify_online_func(specs.OnlineSoftmax()) == "softmax"
    assert identify_online_func(specs.OnlineSoftmaxRespelled()) == "softmax"
    assert identify_online_func(specs.OnlineIdentity()) == "identity"
    assert identify_online_func(specs.OnlineRetention()) == "retention"

    class NoClamp(specs.OnlineRetention):          # differs from the library row function: no clamp
        @staticmethod
        def online_fwd(scores, st, b, h, q_idx):
            r_wo = st["r_wo_clamp"] + scores.get_reduce("abssum")
            return scores / r_wo, {"r_wo_clamp": r_wo, "r": r_wo}, st["r"] / r_wo

    with pytest.raises(NotImplementedError):
        identify_online_func(NoClamp())

    class WrongInit(specs.OnlineSoftmax):
        def __init__(self):
            OnlineFunc.__init__(self, {"m": SymbolScalar("m", Var("0.0")), "r": SymbolScalar("r", Var("0.0"))}, {}, CustomIO())

    with pytest.raises(NotImplementedError):
        identify_online_func(WrongInit())


def test_softmax_with_an_inner_scale_and_no_online_function():
    """The spellings of the reference's second set of examples (examples/mha_v2.py:26-83, sigmoid_attn_v2.py:67): a
    softmax that scales the raw scores itself is the library's softmax of scale * score; None is the identity."""
    scale = (1 / 128) ** 0.5
    name, inner = identify_online_func(specs.online_softmax_inner_scale(scale), return_scale=True)
    assert name == "softmax" and abs(inner - scale) < 1e-12
    assert identify_online_func(specs.OnlineSoftmax(), return_scale=True) == ("softmax", 1.0)
    with pytest.raises(NotImplementedError):          # (a caller that does not ask for the scale must not lose it)
        identify_online_func(specs.online_softmax_inner_scale(scale))
    assert identify_online_func(None) == "identity" and identify_online_func(None, return_scale=True) == ("identity", 1.0)

    e = specs.softmax_attention_inner_scale(2, 4, 256, 128, 128)
    assert (e.family, e.mask_kind) == ("softmax", "causal") and abs(e.score_form.scale - scale) < 1e-12 and e.score_form.bias == 0.0
    # a constant inside the score function is scaled with it: softmax(scale * (2 s + 3))
    e = specs.softmax_attention_inner_scale(2, 4, 256, 128, 128, score_mod=lambda s, c, b, h, q, k: s * 2.0 + 3.0)
    assert abs(e.score_form.scale - 2 * scale) < 1e-12 and abs(e.score_form.bias - 3 * scale) < 1e-12
    # additive tensors would have to be scaled too: refused, not silently left unscaled
    io = CustomIO({"rel": (1, "heads", "seq_len", "seq_len_kv")})
    with pytest.raises(NotImplementedError):
        specs.softmax_attention_inner_scale(2, 4, 256, 128, 128, io=io,
                                            score_mod=lambda s, c, b, h, q, k: s + c.input_tensors["rel"])

    # the recomputation must carry the same scale: exp(s - lse) is another function
    inner_cls = type(specs.online_softmax_inner_scale(scale))

    class ForgetsTheScale(inner_cls):
        @staticmethod
        def forward(scores, final_rowscales, b, h, q_idx, kv_idx):
            return (scores - final_rowscales["lse"]).exp()

    with pytest.raises(NotImplementedError):
        identify_online_func(ForgetsTheScale(), return_scale=True)

    class InconsistentLse(inner_cls):          # lse without the scale on the maximum
        @staticmethod
        def online_fwd_epilogue(o, online_rowscales, b, h, q_idx):
            return o / online_rowscales["r"], {"lse": online_rowscales["r"].log() + online_rowscales["m"]}

    with pytest.raises(NotImplementedError):
        identify_online_func(InconsistentLse(), return_scale=True)

    assert specs.sigmoid_attention(1, 2, 256, 128, 128, online=None).family == "sigmoid"


def test_engine_construction_and_dispatch():
    assert get_attn_device().name == "MI355X"
    e = specs.softmax_attention(8, 32, 4096, 128, 128)
    assert (e.family, e.mask_kind, e.tl_code, e.block_mask) == ("softmax", "causal", "", None)
    assert abs(e.score_form.scale - 128 ** -0.5) < 1e-12
    assert specs.softmax_attention(1, 4, 512, 64, 64, causal=False, online=specs.OnlineSoftmaxRespelled()).mask_kind == "none"
    e = specs.sigmoid_attention(1, 2, 256, 128, 128, scale=128 ** -0.5, const_bias=-math.log(256), form="exp")
    assert e.family == "sigmoid" and abs(e.score_form.bias + math.log(256)) < 1e-9 and e.score_form.bias_tensor is None
    assert specs.sigmoid_attention(1, 2, 256, 128, 128).score_form.bias_tensor == "softmax_bias"
    assert specs.relu_attention(1, 6, 256, 64, 64).family == "relu"
    e = specs.retention_parallel(1, 4, 256, 256, 512)
    assert (e.family, e.score_form.mask_tensor, e.mask_kind) == ("retention", "mask", "causal")
    e = specs.mla_decode(2, 128, 1024, 576, 512)
    assert (e.mla_dim, e.mla_pe) == (512, 64) and abs(e.mla_scale - 576 ** -0.5) < 1e-12
    with pytest.raises(KeyError):                      # fp32 is rejected like the reference's dtype map does
        specs.softmax_attention(1, 4, 512, 64, 64, dtype=torch.float32)
    with pytest.raises(NotImplementedError):           # softmax score with identity row function: not in the library
        AttentionEngine(specs._meta(1, 2, 64, 128, 128, torch.bfloat16), CustomIO({}), score_mod=lambda s, c, b, h, q, k: s * 0.1,
                        mask_mod=None, online_func=specs.OnlineIdentity())
    e = AttentionEngine(specs._meta(1, 8, 64, 128, 128, torch.bfloat16, HKV=2), CustomIO({}),                # grouped-query prefill
                        score_mod=lambda s, c, b, h, q, k: s * 0.1, mask_mod=None, online_func=specs.OnlineSoftmax())
    assert (e.family, e.meta["Hq"], e.meta["Hkv"]) == ("softmax", 8, 2)
    with pytest.raises(NotImplementedError):           # 8 query heads cannot share 3 kv heads
        AttentionEngine(specs._meta(1, 8, 64, 128, 128, torch.bfloat16, HKV=3), CustomIO({}), score_mod=lambda s, c, b, h, q, k: s * 0.1,
                        mask_mod=None, online_func=specs.OnlineSoftmax())


def test_linear_engine_plans():
    p = specs.retnet_recurrent(1, 2, 256, 256, 512).plan
    assert (p.q_scale, p.decay_kind, p.v_scale_tensor) == (256 ** -0.5, "log", None)
    p = specs.gated_retention(1, 2, 256, 256, 256).plan
    assert (p.q_scale, p.decay_kind) == (256 ** -0.5, "identity")
    p = specs.mamba2(1, 1, 256, 128, 64, HK=1, HV=8).plan
    assert (p.q_scale, p.decay_kind, p.decay_head_tensor, p.v_scale_tensor) == (1.0, "mul_head", "A", "dt")
    from attn_engine import LinearAttentionEngine
    e = LinearAttentionEngine(specs._meta(1, 2, 64, 64, 64, torch.bfloat16), k_mod=lambda k, io: k * 0.5,
                              v_mod=lambda v, io: v / 4, decay_mod=lambda d, io: (d * 2.0).log(), custom_io=CustomIO({}))
    assert e.plan.q_scale == 0.125 and e.plan.decay_kind == "traced"
    g = e._log_decay(torch.full((1, 2, 64), 0.25), {})
    torch.testing.assert_close(g, torch.full((1, 2, 64), math.log(0.5)))
    with pytest.raises(NotImplementedError):
        LinearAttentionEngine(specs._meta(1, 2, 64, 64, 64, torch.bfloat16), q_mod=lambda q, io: q.exp(), custom_io=CustomIO({}))
    with pytest.raises(KeyError):
        specs.retnet_recurrent(1, 2, 64, 64, 64, dtype=torch.float16)


def test_operators_refuse_cpu_tensors():
    """No CPU fallback: calling an operator without GPU tensors / library fails loudly."""
    e = specs.softmax_attention(1, 2, 64, 128, 128)
    q = torch.zeros(1, 64, 2, 128, dtype=torch.bfloat16)
    with pytest.raises(Exception) as ei:
        e(q, q, q)
    assert "GPU" in str(ei.value) or "not found" in str(ei.value)


# ------------------------------------------------------------------ spec interpreter vs oracle
@pytest.mark.parametrize("block_n", [0, 1, 7, 64])
def test_c1_softmax_fp32_spec_on_cpu(block_n):
    """B=1 H=4 S=512 D=64 non-causal fp32 (the CPU 'plumbing' configuration): the traced
    spec, run literally tile by tile, equals the oracle for any kv block size."""
    cfg = inputs.CONFIGS["c1_softmax_fp32"]
    S = cfg["S"] if block_n in (0, 64) else 96
    q, k, v = inputs.softmax_inputs(cfg["B"], cfg["H"], S, cfg["D"], cfg["DV"], dtype=torch.float32)
    scale = cfg["D"] ** -0.5
    o, fin = attention_by_spec(q, k, v, [], score_mod=lambda s, c, b, h, qi, ki: s * scale, mask_mod=None,
                               online_func=specs.OnlineSoftmax(), custom_fwd_inputs=CustomIO({}), block_n=block_n)
    ref, lse = oracle.softmax_attention(q, k, v, causal=False, return_lse=True)
    torch.testing.assert_close(o, ref, rtol=2e-5, atol=2e-5)
    torch.testing.assert_close(fin["lse"], lse, rtol=2e-5, atol=2e-5)


@pytest.mark.parametrize("block_n", [0, 16])
def test_specs_on_cpu_match_oracle(block_n):
    B, H, S, D = 1, 2, 48, 16
    q, k, v = inputs.softmax_inputs(B, H, S, D, D, dtype=torch.float32, seed=3)
    cm = specs.causal_mask
    o, _ = attention_by_spec(q, k, v, [], score_mod=lambda s, c, b, h, qi, ki: s * 0.25, mask_mod=cm,
                             online_func=specs.OnlineSoftmaxRespelled(), custom_fwd_inputs=CustomIO({}), block_n=block_n)
    torch.testing.assert_close(o, oracle.softmax_attention(q, k, v, causal=True, softmax_scale=0.25), rtol=2e-5, atol=2e-5)
    io = CustomIO({"softmax_bias": (1,)})
    bias = torch.tensor([-1.5])
    o, _ = attention_by_spec(q, k, v, [bias], mask_mod=cm, online_func=specs.OnlineIdentity(), custom_fwd_inputs=io, block_n=block_n,
                             score_mod=lambda s, c, b, h, qi, ki: (((s + c.input_tensors["softmax_bias"]) * 0.5).tanh() + 1) * 0.5)
    torch.testing.assert_close(o, oracle.sigmoid_attention(q, k, v, bias, causal=True), rtol=2e-5, atol=2e-5)
    io = CustomIO({"mask": (1, "heads", "seq_len", "seq_len_kv")})
    mask = oracle.retention_decay_mask(H, S)
    o, fin = attention_by_spec(q, k, v, [mask], mask_mod=cm, mask_value="0", online_func=specs.OnlineRetention(),
                               custom_fwd_inputs=io, block_n=block_n,
                               score_mod=lambda s, c, b, h, qi, ki: s * c.input_tensors["mask"])
    ref, r = oracle.retention_parallel(q, k, v, mask, return_r=True)
    torch.testing.assert_close(o, ref, rtol=2e-5, atol=2e-5)
    torch.testing.assert_close(fin["r"], r, rtol=2e-5, atol=2e-5)


def test_spec_forward_backward_combine_are_checked_against_the_library():
    """forward / backward / combine of an OnlineFunc are traced and compared with the one version the kernel library
    holds per row function (the spellings of examples/mha.py:73-83, examples/mha_decode.py:72-80 and
    examples/retention_parallel.py:76-86 pass); a spec that defines another one is refused, not silently replaced."""
    class Softmax(specs.OnlineSoftmax):
        @staticmethod
        def forward(scores, final_rowscales, b, h, q_idx, kv_idx):
            return (scores - final_rowscales["lse"]).exp()

        @staticmethod
        def backward(dp, scores, final_rowscales, doosum_rowscales, b, h, q_idx, kv_idx):
            return (dp - doosum_rowscales) * scores

        @staticmethod
        def combine(final_rowscales):
            lse = final_rowscales["lse"]
            lse_max = lse.get_reduce("max")
            row_sum = (lse - lse_max).exp2()
            lse_sum = row_sum.get_reduce("sum").log2() + lse_max
            return (lse - lse_sum).exp2()

    assert identify_online_func(Softmax()) == "softmax"

    class NaturalCombine(Softmax):
        @staticmethod
        def combine(final_rowscales):
            lse = final_rowscales["lse"]
            m = lse.get_reduce("max")
            e = (lse - m).exp()
            return e / e.get_reduce("sum")

    assert identify_online_func(NaturalCombine()) == "softmax"

    class Retention(specs.OnlineRetention):
        @staticmethod
        def forward(scores, final_rowscales, b, h, q_idx, kv_idx):
            return scores / final_rowscales["r"]

        @staticmethod
        def backward(dp, scores, final_rowscales, doosum_rowscales, b, h, q_idx, kv_idx):
            return dp / final_rowscales["r"]

    assert identify_online_func(Retention()) == "retention"

    class WrongBackward(Softmax):
        @staticmethod
        def backward(dp, scores, final_rowscales, doosum_rowscales, b, h, q_idx, kv_idx):
            return dp * scores

    class WrongForward(Softmax):
        @staticmethod
        def forward(scores, final_rowscales, b, h, q_idx, kv_idx):
            return (scores - final_rowscales["lse"]).exp2()

    class WrongCombine(Softmax):
        @staticmethod
        def combine(final_rowscales):
            lse = final_rowscales["lse"]
            return (lse - lse.get_reduce("max")).exp()

    class RetentionTrueGradient(Retention):
        @staticmethod
        def backward(dp, scores, final_rowscales, doosum_rowscales, b, h, q_idx, kv_idx):
            return (dp - doosum_rowscales) / final_rowscales["r"]

    for bad, word in ((WrongBackward, "backward"), (WrongForward, "forward"), (WrongCombine, "combine"), (RetentionTrueGradient, "backward")):
        with pytest.raises(NotImplementedError) as ei:
            identify_online_func(bad())
        assert word in str(ei.value)


def test_bench_refuses_more_than_one_gpu():
    """bench.py --gpus N with N > 1 exits with a message (the build uses one GPU); decided before anything touches a GPU."""
    import os
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    r = subprocess.run([sys.executable, os.path.join(root, "bench.py"), "--gpus", "2"], capture_output=True, text=True, timeout=120, cwd=root)
    assert r.returncode != 0 and "one gpu" in (r.stderr + r.stdout).lower()
