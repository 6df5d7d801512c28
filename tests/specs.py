"""User-level specs written against the public API, in the style of the
reference's examples/ directory (examples/mha.py, sigmoid_attn.py, reluattn.py,
retention_parallel.py, retnet_recurrent.py, mamba2.py, gated_retention.py,
mla_decode.py).  They are what a user of the reference would write; several
use alternative but equivalent spellings to exercise the canonicaliser."""
import torch

from attn_engine import AttentionEngine, LinearAttentionEngine, OnlineFunc
from core import CustomIO, SymbolScalar, Var, meta_tensor
from autotuner.arch import get_attn_device


def causal_mask(b, h, q_idx, kv_idx):
    return q_idx >= kv_idx


class OnlineSoftmax(OnlineFunc):
    def __init__(self):
        super().__init__({"m": SymbolScalar("m", Var("-inf")), "r": SymbolScalar("r", Var("0.0"))},
                         {"lse": SymbolScalar("lse", Var("0.0"))}, CustomIO())

    @staticmethod
    def online_fwd(scores, online_rowscales, b, h, q_idx):
        m, r = online_rowscales["m"], online_rowscales["r"]
        m_new = m.max(scores.get_reduce("max"))
        scale_tmp = (m - m_new).exp()
        r = r * scale_tmp
        scores = (scores - m_new).exp()
        r = r + scores.get_reduce("sum")
        return scores, {"m": m_new, "r": r}, scale_tmp

    @staticmethod
    def online_fwd_epilogue(o, online_rowscales, b, h, q_idx):
        lse = online_rowscales["r"].log() + online_rowscales["m"]
        return o / online_rowscales["r"], {"lse": lse}


class OnlineSoftmaxRespelled(OnlineFunc):
    """Same row function, different variable names / operand order."""

    def __init__(self):
        super().__init__({"denom": SymbolScalar("denom", Var("0.0")), "peak": SymbolScalar("peak", Var("-inf"))},
                         {"logsum": SymbolScalar("logsum", Var("0.0"))}, CustomIO())

    @staticmethod
    def online_fwd(scores, st, b, h, q_idx):
        peak = scores.get_reduce("max").max(st["peak"])
        corr = (st["peak"] - peak).exp()
        p = (scores - peak).exp()
        denom = p.get_reduce("sum") + corr * st["denom"]
        return p, {"peak": peak, "denom": denom}, corr

    @staticmethod
    def online_fwd_epilogue(o, st, b, h, q_idx):
        return o / st["denom"], {"logsum": st["peak"] + st["denom"].log()}


def online_softmax_inner_scale(scale):
    """A softmax that scales the raw scores itself, in base 2 (the spelling of examples/mha_v2.py:26-83): the running
    maximum is kept in the units of the raw scores, lse = log r + scale * m."""
    import math
    sl2 = scale * math.log2(math.e)

    class OnlineSoftmaxInnerScale(OnlineFunc):
        def __init__(self):
            super().__init__({"m": SymbolScalar("m", Var("-inf")), "r": SymbolScalar("r", Var("0.0"))},
                             {"lse": SymbolScalar("lse", Var("0.0"))}, CustomIO())

        @staticmethod
        def online_fwd(scores, online_rowscales, b, h, q_idx):
            m, r = online_rowscales["m"], online_rowscales["r"]
            m_new = m.max(scores.get_reduce("max"))
            scale_tmp = ((m - m_new) * sl2).exp2()
            r = r * scale_tmp
            scores = ((scores - m_new) * sl2).exp2()
            r = r + scores.get_reduce("sum")
            return scores, {"m": m_new, "r": r}, scale_tmp

        @staticmethod
        def online_fwd_epilogue(o, online_rowscales, b, h, q_idx):
            lse = online_rowscales["r"].log() + online_rowscales["m"] * scale
            return o / online_rowscales["r"], {"lse": lse}

        @staticmethod
        def forward(scores, final_rowscales, b, h, q_idx, kv_idx):
            return (scores * scale - final_rowscales["lse"]).exp()

        @staticmethod
        def backward(dp, scores, final_rowscales, doosum_rowscales, b, h, q_idx, kv_idx):
            return (dp - doosum_rowscales) * scores

    return OnlineSoftmaxInnerScale()


class OnlineIdentity(OnlineFunc):
    def __init__(self):
        super().__init__({}, {}, CustomIO())

    @staticmethod
    def online_fwd(scores, online_rowscales, b, h, q_idx):
        return scores, online_rowscales, SymbolScalar("o_scale", Var("1"))

    @staticmethod
    def online_fwd_epilogue(o, online_rowscales, b, h, q_idx):
        return o, {}


class OnlineRetention(OnlineFunc):
    def __init__(self):
        super().__init__({"r_wo_clamp": SymbolScalar("r_wo_clamp", Var("0.0")), "r": SymbolScalar("r", Var("0.0"))},
                         {"r": SymbolScalar("r", Var("0.0"))}, CustomIO())

    @staticmethod
    def online_fwd(scores, online_rowscales, b, h, q_idx):
        r_wo_clamp = online_rowscales["r_wo_clamp"] + scores.get_reduce("abssum")
        r_new = r_wo_clamp.max(1.0)
        o_scale = online_rowscales["r"] / r_new
        return scores / r_new, {"r_wo_clamp": r_wo_clamp, "r": r_new}, o_scale

    @staticmethod
    def online_fwd_epilogue(o, online_rowscales, b, h, q_idx):
        return o, {"r": online_rowscales["r"]}


def _meta(B, H, S, D, DV, dtype, SKV=None, HKV=None):
    return (meta_tensor(B, H, S, D, dtype=dtype), meta_tensor(B, HKV or H, SKV or S, D, dtype=dtype),
            meta_tensor(B, HKV or H, SKV or S, DV, dtype=dtype))


def softmax_attention(B, H, S, D, DV, dtype=torch.bfloat16, causal=True, online=None, tune=False):
    scale = 1 / D ** 0.5

    def score_mod(score, custom_fwd_inputs, b, h, q_idx, kv_idx):
        return score * scale

    dev = get_attn_device()
    return AttentionEngine(_meta(B, H, S, D, DV, dtype), CustomIO({}), score_mod=score_mod,
                           mask_mod=causal_mask if causal else None, online_func=online or OnlineSoftmax(),
                           tune=tune, tune_file=f"tuned_config/{dev.name}/attn_tl.json", infer_mask=True)


def softmax_attention_inner_scale(B, H, S, D, DV, dtype=torch.bfloat16, causal=True, score_mod=None, io=None):
    """examples/mha_v2.py:15-99: the score_mod returns the raw score, the online function scales it."""
    if score_mod is None:
        def score_mod(score, custom_fwd_inputs, b, h, q_idx, kv_idx):
            return score
    return AttentionEngine(_meta(B, H, S, D, DV, dtype), io or CustomIO({}), score_mod=score_mod,
                           mask_mod=causal_mask if causal else None, online_func=online_softmax_inner_scale((1 / D) ** 0.5),
                           backend="cute_v2")


def sigmoid_attention(B, H, S, D, DV, dtype=torch.bfloat16, scale=1.0, form="tanh", const_bias=None, causal=True, mask_mod=None,
                      online="identity"):
    def score_mod(score, custom_fwd_inputs, b, h, q_idx, kv_idx):
        x = score * scale if scale != 1.0 else score
        x = x + (const_bias if const_bias is not None else custom_fwd_inputs.input_tensors["softmax_bias"])
        if form == "tanh":
            return ((x * 0.5).tanh() + 1) * 0.5
        return 1 / (1 + (-x).exp())

    io = CustomIO({} if const_bias is not None else {"softmax_bias": (1,)})
    return AttentionEngine(_meta(B, H, S, D, DV, dtype), io, score_mod=score_mod,
                           mask_mod=mask_mod if mask_mod is not None else (causal_mask if causal else None),
                           online_func=OnlineIdentity() if online == "identity" else online)


def relu_attention(B, H, S, D, DV, dtype=torch.bfloat16):
    scale = 1 / D ** 0.5

    def score_mod(score, custom_fwd_inputs, b, h, q_idx, kv_idx):
        return (score * scale).max(0)

    return AttentionEngine(_meta(B, H, S, D, DV, dtype), CustomIO({}), score_mod=score_mod, mask_mod=None,
                           online_func=OnlineIdentity())


def retention_parallel(B, H, S, D, DV, dtype=torch.bfloat16):
    def score_mod(score, custom_fwd_inputs, b, h, q_idx, kv_idx):
        return score * custom_fwd_inputs.input_tensors["mask"]

    io = CustomIO({"mask": (1, "heads", "seq_len", "seq_len_kv")})
    return AttentionEngine(_meta(B, H, S, D, DV, dtype), io, score_mod=score_mod, mask_mod=causal_mask,
                           online_func=OnlineRetention(), mask_value="0")


def mla_decode(B, H, SKV, D, DV, dtype=torch.bfloat16):
    scale = 1 / D ** 0.5

    def score_mod(score, custom_fwd_inputs, b, h, q_idx, kv_idx):
        return score * scale

    meta = (meta_tensor(B, H, 1, D, dtype=dtype), meta_tensor(B, 1, SKV, D, dtype=dtype), meta_tensor(B, 1, SKV, DV, dtype=dtype))
    return AttentionEngine(meta, CustomIO({}), score_mod=score_mod, mask_mod=None, online_func=OnlineSoftmax(), kv_shared=True)


def retnet_recurrent(B, H, S, D, DV, dtype=torch.bfloat16, chunk_size=None):
    scale = 1 / D ** 0.5
    return LinearAttentionEngine(_meta(B, H, S, D, DV, dtype), q_mod=lambda q, io: q * scale,
                                 decay_mod=lambda decay, io: decay.log(), custom_io=CustomIO({}), chunk_size=chunk_size)


def gated_retention(B, H, S, D, DV, dtype=torch.bfloat16, chunk_size=None):
    scale = 1 / D ** 0.5
    return LinearAttentionEngine(_meta(B, H, S, D, DV, dtype), q_mod=lambda q, io: q * scale, custom_io=CustomIO({}),
                                 chunk_size=chunk_size)


def mamba2(B, HQ, S, D, DV, HK=None, HV=None, dtype=torch.bfloat16, chunk_size=None):
    HK, HV = HK or HQ, HV or HQ
    meta = (meta_tensor(B, HQ, S, D, dtype=dtype), meta_tensor(B, HK, S, D, dtype=dtype), meta_tensor(B, HV, S, DV, dtype=dtype))
    io = CustomIO({"A": (1, "heads"), "dt": ("batch", "heads", "seq_len")})
    return LinearAttentionEngine(meta, decay_mod=lambda decay, io: decay * io.input_tensors["A"],
                                 v_mod=lambda v, io: v * io.input_tensors["dt"], custom_io=io, chunk_size=chunk_size)


def softmax_attention_decode(B, H, S, KV, D, DV, dtype=torch.float16, HKV=None):
    """examples/mha_decode.py:14-123: no mask, declared query length padded to a multiple of 128."""
    scale = 1 / D ** 0.5
    HKV = HKV or H
    meta = (meta_tensor(B, H, ((S + 127) // 128) * 128, D, dtype=dtype), meta_tensor(B, HKV, KV, D, dtype=dtype),
            meta_tensor(B, HKV, KV, DV, dtype=dtype))
    return AttentionEngine(meta, CustomIO({}), score_mod=lambda score, io, b, h, q_idx, kv_idx: score * scale, mask_mod=None,
                           online_func=OnlineSoftmax())


def sparse_gqa_decode(B, H, G, S, D, DV, dtype=torch.float16, block=32):
    """examples/sparse_gqa_decode.py:13-107: one query token, G kv heads, external kv block mask and per-batch cache lengths."""
    scale = 1 / D ** 0.5
    meta = (meta_tensor(B, H, 1, D, dtype=dtype), meta_tensor(B, G, S, D, dtype=dtype), meta_tensor(B, G, S, DV, dtype=dtype))
    return AttentionEngine(meta, CustomIO({}), score_mod=lambda score, io, b, h, q_idx, kv_idx: score * scale, mask_mod=None,
                           online_func=OnlineSoftmax(), extern_block_mask=True, use_varlen=True, infer_mask_block_N=block)
