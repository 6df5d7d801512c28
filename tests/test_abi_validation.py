"""Argument checking of the C ABI, without a GPU: every entry point checks what it is given before it touches the device,
so bad arguments come back as MA_ERR_INVALID_ARG / MA_ERR_UNSUPPORTED / MA_ERR_WORKSPACE with a message, never as a crash
or a launch.  The pointers here are made-up addresses that nothing may dereference; an argument set that is valid gets as
far as the launch and fails there (MA_ERR_LAUNCH) because this test only runs where there is no GPU."""
import ctypes

import pytest
import torch

from metaattention_amd import hip_backend as hb

pytestmark = pytest.mark.skipif(torch.cuda.is_available(), reason="made-up pointers: only where no kernel can be launched")

INVALID, UNSUPPORTED, WORKSPACE, LAUNCH = -1, -2, -3, -4
PTR = 0x7F0000000000


def _lib():
    return hb.load_library()


def _attn(**over):
    p = hb.AttnParams()
    p.family, p.dtype, p.mask = hb.MA_ATTN_SOFTMAX, hb.MA_BF16, hb.MA_MASK_CAUSAL
    p.batch, p.heads, p.heads_kv, p.seqlen_q, p.seqlen_kv, p.dim_qk, p.dim_v = 2, 4, 4, 256, 256, 128, 128
    for i, name in enumerate(("q", "k", "v", "o")):
        setattr(p, name, PTR + i * 0x10000000)
        setattr(p, f"{name}_stride_b", 256 * 4 * 128)
        setattr(p, f"{name}_stride_s", 4 * 128)
        setattr(p, f"{name}_stride_h", 128)
    p.scale = 0.088
    for key, val in over.items():
        setattr(p, key, val)
    return p


def _attn_bwd(**over):
    p = hb.AttnBwdParams()
    p.family, p.dtype, p.mask = hb.MA_ATTN_SOFTMAX, hb.MA_BF16, hb.MA_MASK_CAUSAL
    p.batch, p.heads, p.heads_kv, p.seqlen_q, p.seqlen_kv, p.dim_qk, p.dim_v = 2, 4, 4, 256, 256, 128, 128
    for i, name in enumerate(("q", "k", "v", "o", "dq", "dk", "dv")):
        setattr(p, name, PTR + i * 0x10000000)
        setattr(p, f"{name}_stride_b", 256 * 4 * 128)
        setattr(p, f"{name}_stride_s", 4 * 128)
        setattr(p, f"{name}_stride_h", 128)
    p.dout, p.do_stride_b, p.do_stride_s, p.do_stride_h = PTR + 0x80000000, 256 * 4 * 128, 4 * 128, 128
    p.lse = PTR + 0x90000000
    p.scale = 0.088
    p.workspace, p.workspace_bytes = PTR + 0xA0000000, 1 << 30
    for key, val in over.items():
        setattr(p, key, val)
    return p


def _linear(**over):
    p = hb.LinearParams()
    p.dtype, p.batch, p.heads, p.heads_q, p.heads_k, p.seqlen, p.dim_k, p.dim_v = hb.MA_BF16, 2, 4, 4, 4, 256, 128, 128
    p.q, p.k, p.v, p.o, p.log_decay = (PTR + i * 0x10000000 for i in range(5))
    p.q_scale = 1.0
    for key, val in over.items():
        setattr(p, key, val)
    return p


def _linear_bwd(**over):
    p = hb.LinearBwdParams()
    p.dtype, p.batch, p.heads, p.heads_q, p.heads_k, p.seqlen, p.dim_k, p.dim_v = hb.MA_BF16, 2, 4, 4, 4, 256, 128, 128
    p.q, p.k, p.v, p.dout, p.log_decay, p.dq, p.dk, p.dv, p.dlog_decay = (PTR + i * 0x10000000 for i in range(9))
    p.q_scale = 1.0
    p.workspace, p.workspace_bytes = PTR + 0xA0000000, 1 << 34
    for key, val in over.items():
        setattr(p, key, val)
    return p


def _mla(**over):
    p = hb.MlaParams()
    p.dtype, p.batch, p.heads_q, p.seqlen_kv, p.dim, p.dim_pe, p.num_split = hb.MA_BF16, 2, 128, 1024, 512, 64, 1
    p.q, p.q_stride_b, p.q_stride_h = PTR, 128 * 512, 512
    p.q_pe, p.qpe_stride_b, p.qpe_stride_h = PTR + 0x10000000, 128 * 64, 64
    p.kv, p.kv_stride_b, p.kv_stride_s = PTR + 0x20000000, 1024 * 512, 512
    p.k_pe, p.kpe_stride_b, p.kpe_stride_s = PTR + 0x30000000, 1024 * 64, 64
    p.o, p.o_stride_b, p.o_stride_h = PTR + 0x40000000, 128 * 512, 512
    p.scale = 0.0417
    for key, val in over.items():
        setattr(p, key, val)
    return p


CASES = [
    # ---- ma_attn_fwd
    ("ma_attn_fwd", _attn, {}, LAUNCH),
    ("ma_attn_fwd", _attn, {"q": None}, INVALID), ("ma_attn_fwd", _attn, {"o": None}, INVALID),
    ("ma_attn_fwd", _attn, {"batch": 0}, INVALID), ("ma_attn_fwd", _attn, {"seqlen_kv": -3}, INVALID), ("ma_attn_fwd", _attn, {"dim_v": 0}, INVALID),
    ("ma_attn_fwd", _attn, {"dtype": 7}, INVALID), ("ma_attn_fwd", _attn, {"mask": 5}, INVALID), ("ma_attn_fwd", _attn, {"family": 11}, INVALID),
    ("ma_attn_fwd", _attn, {"scale": 0.0}, INVALID), ("ma_attn_fwd", _attn, {"scale": float("nan")}, INVALID),
    ("ma_attn_fwd", _attn, {"seqlen_kv": 300}, UNSUPPORTED),                    # causal with unequal lengths
    ("ma_attn_fwd", _attn, {"heads_kv": 3}, INVALID),
    ("ma_attn_fwd", _attn, {"dim_qk": 96, "dim_v": 96}, UNSUPPORTED), ("ma_attn_fwd", _attn, {"dim_qk": 128, "dim_v": 64}, UNSUPPORTED),
    ("ma_attn_fwd", _attn, {"q_stride_s": 4 * 128 + 4}, UNSUPPORTED), ("ma_attn_fwd", _attn, {"k": PTR + 8}, UNSUPPORTED),
    ("ma_attn_fwd", _attn, {"kv_block_mask": PTR + 0x50000000, "kv_block_size": 48, "mask": hb.MA_MASK_NONE}, UNSUPPORTED),
    ("ma_attn_fwd", _attn, {"kv_seqlens": PTR + 0x50000000}, UNSUPPORTED),      # cache lengths under the causal mask
    ("ma_attn_fwd", _attn, {"elem_mask": PTR + 0x50000000}, UNSUPPORTED),       # element mask under the causal mask
    ("ma_attn_fwd", _attn, {"elem_mask": PTR + 0x50000000, "mask": hb.MA_MASK_NONE, "em_stride_q": 258}, UNSUPPORTED),
    ("ma_attn_fwd", _attn, {"family": hb.MA_ATTN_RETENTION}, INVALID),          # retention without a multiplier
    ("ma_attn_fwd", _attn, {"family": hb.MA_ATTN_RETENTION, "score_mask": PTR + 0x50000004, "sm_stride_h": 256 * 256, "sm_stride_q": 256}, UNSUPPORTED),
    ("ma_attn_fwd", _attn, {"decay_gamma": PTR + 0x50000000}, UNSUPPORTED),     # decay_gamma outside the retention family
    ("ma_attn_fwd", _attn, {"family": hb.MA_ATTN_RETENTION, "decay_gamma": PTR + 0x50000000}, UNSUPPORTED),   # .. and at 128 / 128
    ("ma_attn_fwd", _attn, {"family": hb.MA_ATTN_SIGMOID, "softcap": 30.0}, UNSUPPORTED), ("ma_attn_fwd", _attn, {"softcap": -1.0}, UNSUPPORTED),
    ("ma_attn_fwd", _attn, {"score_add": PTR + 0x50000002, "score_add_fp32": 1}, UNSUPPORTED),
    # (sizes whose work-item counts leave 32 bits)
    ("ma_attn_fwd", _attn, {"batch": (1 << 31) - 1, "heads": (1 << 31) - 1, "heads_kv": (1 << 31) - 1}, UNSUPPORTED),
    ("ma_attn_fwd", _attn, {"seqlen_q": (1 << 31) - 1, "seqlen_kv": (1 << 31) - 1}, UNSUPPORTED),
    ("ma_attn_fwd", _attn, {"batch": 1 << 20, "seqlen_q": 1 << 20, "seqlen_kv": 1 << 20}, UNSUPPORTED),
    ("ma_attn_fwd", _attn, {"v_stride_s": 1 << 62}, UNSUPPORTED), ("ma_attn_fwd", _attn, {"score_add": PTR + 0x50000000, "v_stride_s": 1 << 62}, UNSUPPORTED),
    ("ma_attn_fwd", _attn, {"elem_mask": PTR + 0x50000000, "mask": hb.MA_MASK_NONE, "em_stride_b": 1 << 62}, UNSUPPORTED),
    # ---- ma_attn_bwd
    ("ma_attn_bwd", _attn_bwd, {}, LAUNCH),
    ("ma_attn_bwd", _attn_bwd, {"dout": None}, INVALID), ("ma_attn_bwd", _attn_bwd, {"dk": None}, INVALID), ("ma_attn_bwd", _attn_bwd, {"heads": 0}, INVALID),
    ("ma_attn_bwd", _attn_bwd, {"lse": None}, INVALID), ("ma_attn_bwd", _attn_bwd, {"o": None}, INVALID),
    ("ma_attn_bwd", _attn_bwd, {"family": 9}, UNSUPPORTED), ("ma_attn_bwd", _attn_bwd, {"scale": -1.0}, INVALID),
    ("ma_attn_bwd", _attn_bwd, {"seqlen_q": 200}, UNSUPPORTED), ("ma_attn_bwd", _attn_bwd, {"heads_kv": 3}, INVALID),
    ("ma_attn_bwd", _attn_bwd, {"workspace": None}, WORKSPACE), ("ma_attn_bwd", _attn_bwd, {"workspace_bytes": 64}, WORKSPACE),
    ("ma_attn_bwd", _attn_bwd, {"dq_stride_s": 4 * 128 + 1}, UNSUPPORTED), ("ma_attn_bwd", _attn_bwd, {"dv": PTR + 0x60000004}, UNSUPPORTED),
    ("ma_attn_bwd", _attn_bwd, {"elem_mask": PTR + 0xB0000000, "mask": hb.MA_MASK_NONE}, INVALID),         # without its transpose
    ("ma_attn_bwd", _attn_bwd, {"elem_mask": PTR + 0xB0000000, "elem_mask_t": PTR + 0xC0000000}, UNSUPPORTED),   # under the causal mask
    ("ma_attn_bwd", _attn_bwd, {"kv_block_mask": PTR + 0xB0000000, "mask": hb.MA_MASK_NONE}, INVALID),     # without q_block_mask
    ("ma_attn_bwd", _attn_bwd, {"kv_block_mask": PTR + 0xB0000000, "q_block_mask": PTR + 0xC0000000, "mask": hb.MA_MASK_NONE}, UNSUPPORTED),
    ("ma_attn_bwd", _attn_bwd, {"family": hb.MA_ATTN_RETENTION}, INVALID),
    ("ma_attn_bwd", _attn_bwd, {"family": hb.MA_ATTN_SIGMOID, "softcap": 5.0}, UNSUPPORTED),
    ("ma_attn_bwd", _attn_bwd, {"dim_qk": 96, "dim_v": 96}, UNSUPPORTED),
    ("ma_attn_bwd", _attn_bwd, {"mask": 65536}, INVALID),
    ("ma_attn_bwd", _attn_bwd, {"batch": 1 << 24, "heads": 1 << 10, "heads_kv": 1 << 10, "workspace_bytes": 1 << 62}, UNSUPPORTED),
    # ---- ma_linear_fwd / ma_linear_bwd
    ("ma_linear_fwd", _linear, {}, LAUNCH),
    ("ma_linear_fwd", _linear, {"seqlen": 0}, INVALID), ("ma_linear_fwd", _linear, {"log_decay": None}, INVALID), ("ma_linear_fwd", _linear, {"q": None}, INVALID),
    ("ma_linear_fwd", _linear, {"dtype": hb.MA_FP16}, UNSUPPORTED), ("ma_linear_fwd", _linear, {"heads_q": 3}, INVALID),
    ("ma_linear_fwd", _linear, {"segments": -1}, INVALID), ("ma_linear_fwd", _linear, {"dim_k": 96}, UNSUPPORTED),
    ("ma_linear_fwd", _linear, {"dim_v": 96}, UNSUPPORTED), ("ma_linear_fwd", _linear, {"v": PTR + 0x20000002}, UNSUPPORTED),
    ("ma_linear_fwd", _linear, {"batch": 1 << 20, "heads": 1 << 10, "heads_q": 1 << 10, "heads_k": 1 << 10}, UNSUPPORTED),   # grid too large
    ("ma_linear_fwd", _linear, {"batch": (1 << 31) - 1, "heads": (1 << 31) - 1, "heads_q": (1 << 31) - 1, "heads_k": (1 << 31) - 1, "dim_v": 1 << 30}, UNSUPPORTED),
    ("ma_linear_fwd", _linear, {"seqlen": (1 << 31) - 1}, UNSUPPORTED), ("ma_linear_fwd", _linear, {"dim_v": (1 << 31) - 1}, UNSUPPORTED),
    ("ma_linear_bwd", _linear_bwd, {}, LAUNCH),
    ("ma_linear_bwd", _linear_bwd, {"batch": (1 << 31) - 1, "heads": (1 << 31) - 1, "heads_q": (1 << 31) - 1, "heads_k": (1 << 31) - 1, "seqlen": (1 << 31) - 1}, UNSUPPORTED),
    ("ma_linear_bwd", _linear_bwd, {"dlog_decay": None}, INVALID), ("ma_linear_bwd", _linear_bwd, {"heads_k": 3}, INVALID),
    ("ma_linear_bwd", _linear_bwd, {"dim_k": 320}, UNSUPPORTED), ("ma_linear_bwd", _linear_bwd, {"dim_v": 8192}, UNSUPPORTED),
    ("ma_linear_bwd", _linear_bwd, {"workspace": None}, WORKSPACE), ("ma_linear_bwd", _linear_bwd, {"workspace_bytes": 1024}, WORKSPACE),
    ("ma_linear_bwd", _linear_bwd, {"workspace": PTR + 0xA0000010}, WORKSPACE), ("ma_linear_bwd", _linear_bwd, {"dq": PTR + 0x50000008}, UNSUPPORTED),
    # ---- ma_mla_decode
    ("ma_mla_decode", _mla, {}, LAUNCH),
    ("ma_mla_decode", _mla, {"k_pe": None}, INVALID), ("ma_mla_decode", _mla, {"heads_q": 0}, INVALID), ("ma_mla_decode", _mla, {"dtype": 3}, INVALID),
    ("ma_mla_decode", _mla, {"scale": 0.0}, INVALID), ("ma_mla_decode", _mla, {"batch": 70000}, UNSUPPORTED),
    ("ma_mla_decode", _mla, {"kv_stride_s": 516}, UNSUPPORTED), ("ma_mla_decode", _mla, {"q_pe": PTR + 0x10000008}, UNSUPPORTED),
    ("ma_mla_decode", _mla, {"num_split": 17}, INVALID),                         # more splits than 64-row tiles
    ("ma_mla_decode", _mla, {"num_split": 4}, WORKSPACE),                        # splits without a workspace
    ("ma_mla_decode", _mla, {"num_split": 4, "workspace": PTR + 0x50000000, "workspace_bytes": 4096}, WORKSPACE),
    ("ma_mla_decode", _mla, {"dim": 256, "dim_pe": 32}, UNSUPPORTED),
    ("ma_mla_decode", _mla, {"batch": 65535, "heads_q": 1 << 24, "num_split": 0}, UNSUPPORTED),      # (batch x blocks of heads leaves 32 bits)
    ("ma_mla_decode", _mla, {"seqlen_kv": (1 << 31) - 1}, UNSUPPORTED), ("ma_mla_decode", _mla, {"kv_stride_s": 1 << 62}, UNSUPPORTED),
    ("ma_mla_decode", _mla, {"block_table": PTR + 0x50000000, "block_table_stride": 1 << 62, "page_size": 64}, INVALID),
    ("ma_mla_decode", _mla, {"block_table": PTR + 0x50000000, "block_table_stride": 16, "page_size": 48}, UNSUPPORTED),
    ("ma_mla_decode", _mla, {"block_table": PTR + 0x50000000, "block_table_stride": 4, "page_size": 64}, INVALID),    # rows do not cover the cache
    ("ma_mla_decode", _mla, {"tile_scheduler_metadata": PTR + 0x50000000}, INVALID),     # a plan without its split table
]


@pytest.mark.parametrize("entry,make,over,want", CASES, ids=[f"{c[0]}-{i}" for i, c in enumerate(CASES)])
def test_argument_checks(entry, make, over, want):
    lib = _lib()
    rc = getattr(lib, entry)(ctypes.byref(make(**over)), None)
    msg = lib.ma_last_error().decode()
    assert rc == want, (rc, msg)
    assert msg.startswith(entry + ":") or msg.startswith("ma_linear"), msg


def test_workspace_queries_take_bad_arguments():
    lib = _lib()
    assert lib.ma_linear_workspace_bytes(ctypes.byref(_linear(seqlen=0))) == 0
    assert lib.ma_linear_workspace_bytes(None) == 0
    assert lib.ma_attn_bwd_workspace_bytes(None) == 0
    assert lib.ma_mla_workspace_bytes(None) == 0
    assert lib.ma_mla_workspace_bytes(ctypes.byref(_mla(num_split=4))) >= 2 * 4 * 128 * 512 * 2
    # the split choice divides the CUs by batch x blocks of heads: a product beyond 32 bits must not wrap to zero
    assert lib.ma_mla_choose_split(ctypes.byref(_mla(batch=1 << 20, heads_q=1 << 24, num_split=0))) == 1
    assert lib.ma_mla_choose_split(ctypes.byref(_mla(batch=65535, heads_q=(1 << 31) - 1, num_split=0))) == 1
    assert lib.ma_mla_num_sm_parts((1 << 31) - 1) >= 1 and lib.ma_mla_num_sm_parts(0) == 0
    # sizes whose products leave 64 bits: the queries answer 0 (nothing to allocate for a call that will be refused)
    big = (1 << 31) - 1
    assert lib.ma_attn_workspace_bytes(ctypes.byref(_attn(batch=big, heads=big, heads_kv=big))) == 0
    assert lib.ma_attn_bwd_workspace_bytes(ctypes.byref(_attn_bwd(batch=big, heads=big, heads_kv=big))) == 0
    assert lib.ma_linear_bwd_workspace_bytes(ctypes.byref(_linear_bwd(batch=big, heads=1 << 24, heads_q=4, heads_k=4, seqlen=65536))) == 0
    assert lib.ma_linear_workspace_bytes(ctypes.byref(_linear(dim_v=big))) == 0
    assert lib.ma_mla_workspace_bytes(ctypes.byref(_mla(batch=big, heads_q=big, num_split=4))) == 0
