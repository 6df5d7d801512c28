"""ctypes binding of the gfx950 kernel library (``include/metaattention_hip.h``).

The structures below mirror the C header field by field.  The wrappers take
torch tensors that already live on the GPU, pass raw pointers, strides and the
current HIP stream, and raise ``MetaAttentionError`` carrying the library's
error string when a call is rejected.  There is no fallback: if the shared
library has not been built, loading it raises.
"""
from __future__ import annotations

import ctypes
import os
from ctypes import POINTER, Structure, c_char_p, c_float, c_int, c_int32, c_int64, c_size_t, c_void_p

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(os.path.dirname(_HERE), "lib", "libmetaattention_hip.so")

MA_BF16, MA_FP16 = 0, 1
MA_ATTN_SOFTMAX, MA_ATTN_SIGMOID, MA_ATTN_RELU, MA_ATTN_RETENTION = 0, 1, 2, 3
MA_MASK_NONE, MA_MASK_CAUSAL = 0, 1

EXPORTED_SYMBOLS = (
    "ma_version", "ma_last_error", "ma_attn_workspace_bytes", "ma_attn_fwd", "ma_attn_bwd_workspace_bytes", "ma_attn_bwd",
    "ma_linear_workspace_bytes", "ma_linear_fwd", "ma_linear_bwd_workspace_bytes", "ma_linear_bwd",
    "ma_mla_choose_split", "ma_mla_workspace_bytes", "ma_mla_decode", "ma_mla_num_sm_parts", "ma_mla_get_metadata",
    "ma_mla_noalloc_max_workspace", "ma_mla_decode_noalloc",
)


class MetaAttentionError(RuntimeError):
    def __init__(self, code: int, message: str):
        super().__init__(f"[{code}] {message}")
        self.code = code


class AttnParams(Structure):
    _fields_ = [
        ("family", c_int32), ("dtype", c_int32), ("mask", c_int32),
        ("batch", c_int32), ("heads", c_int32), ("seqlen_q", c_int32), ("seqlen_kv", c_int32),
        ("dim_qk", c_int32), ("dim_v", c_int32),
        ("q", c_void_p), ("q_stride_b", c_int64), ("q_stride_s", c_int64), ("q_stride_h", c_int64),
        ("k", c_void_p), ("k_stride_b", c_int64), ("k_stride_s", c_int64), ("k_stride_h", c_int64),
        ("v", c_void_p), ("v_stride_b", c_int64), ("v_stride_s", c_int64), ("v_stride_h", c_int64),
        ("o", c_void_p), ("o_stride_b", c_int64), ("o_stride_s", c_int64), ("o_stride_h", c_int64),
        ("row_scale", c_void_p),
        ("scale", c_float), ("bias", c_float), ("bias_ptr", c_void_p),
        ("score_mask", c_void_p), ("sm_stride_b", c_int64), ("sm_stride_h", c_int64), ("sm_stride_q", c_int64),
        ("heads_kv", c_int32),
        ("kv_block_size", c_int32), ("kv_seqlens", c_void_p),
        ("kv_block_mask", c_void_p), ("kbm_stride_b", c_int64), ("kbm_stride_h", c_int64),
        ("elem_mask", c_void_p), ("em_stride_b", c_int64), ("em_stride_h", c_int64), ("em_stride_q", c_int64),
        ("kbm_stride_q", c_int64), ("kbm_per_query_head", c_int32),
        ("workspace", c_void_p), ("workspace_bytes", c_size_t),
        ("score_add", c_void_p), ("sa_stride_b", c_int64), ("sa_stride_h", c_int64), ("sa_stride_q", c_int64), ("sa_stride_kv", c_int64),
        ("score_add_fp32", c_int32), ("pos_slope_q", c_void_p), ("pos_slope_kv", c_void_p), ("softcap", c_float),
        ("decay_gamma", c_void_p),
    ]


def _tensor_fields(name):
    return [(name, c_void_p), (f"{name}_stride_b", c_int64), (f"{name}_stride_s", c_int64), (f"{name}_stride_h", c_int64)]


class AttnBwdParams(Structure):
    _fields_ = [
        ("family", c_int32), ("dtype", c_int32), ("mask", c_int32),
        ("batch", c_int32), ("heads", c_int32), ("heads_kv", c_int32), ("seqlen_q", c_int32), ("seqlen_kv", c_int32),
        ("dim_qk", c_int32), ("dim_v", c_int32),
        *_tensor_fields("q"), *_tensor_fields("k"), *_tensor_fields("v"), *_tensor_fields("o"),
        ("dout", c_void_p), ("do_stride_b", c_int64), ("do_stride_s", c_int64), ("do_stride_h", c_int64),
        *_tensor_fields("dq"), *_tensor_fields("dk"), *_tensor_fields("dv"),
        ("lse", c_void_p),
        ("scale", c_float), ("bias", c_float), ("bias_ptr", c_void_p),
        ("workspace", c_void_p), ("workspace_bytes", c_size_t),
        ("elem_mask", c_void_p), ("em_stride_b", c_int64), ("em_stride_h", c_int64), ("em_stride_q", c_int64),
        ("elem_mask_t", c_void_p), ("emt_stride_b", c_int64), ("emt_stride_h", c_int64), ("emt_stride_k", c_int64),
        ("kv_block_mask", c_void_p), ("kbm_stride_b", c_int64), ("kbm_stride_h", c_int64), ("kbm_stride_q", c_int64),
        ("q_block_mask", c_void_p), ("qbm_stride_b", c_int64), ("qbm_stride_h", c_int64), ("qbm_stride_k", c_int64),
        ("score_mask", c_void_p), ("sm_stride_b", c_int64), ("sm_stride_h", c_int64), ("sm_stride_q", c_int64),
        ("score_mask_t", c_void_p), ("smt_stride_b", c_int64), ("smt_stride_h", c_int64), ("smt_stride_k", c_int64),
        ("score_add", c_void_p), ("sa_stride_b", c_int64), ("sa_stride_h", c_int64), ("sa_stride_q", c_int64), ("sa_stride_kv", c_int64),
        ("score_add_fp32", c_int32), ("pos_slope_q", c_void_p), ("pos_slope_kv", c_void_p), ("softcap", c_float),
    ]


class LinearParams(Structure):
    _fields_ = [
        ("dtype", c_int32),
        ("batch", c_int32), ("heads", c_int32), ("heads_q", c_int32), ("heads_k", c_int32),
        ("seqlen", c_int32), ("dim_k", c_int32), ("dim_v", c_int32), ("chunk", c_int32),
        ("q", c_void_p), ("k", c_void_p), ("v", c_void_p), ("o", c_void_p),
        ("log_decay", c_void_p), ("v_scale", c_void_p),
        ("q_scale", c_float), ("segments", c_int32), ("out_fp32", c_int32),
        ("workspace", c_void_p), ("workspace_bytes", c_size_t),
    ]


class LinearBwdParams(Structure):
    _fields_ = [
        ("dtype", c_int32),
        ("batch", c_int32), ("heads", c_int32), ("heads_q", c_int32), ("heads_k", c_int32),
        ("seqlen", c_int32), ("dim_k", c_int32), ("dim_v", c_int32),
        ("q", c_void_p), ("k", c_void_p), ("v", c_void_p), ("dout", c_void_p),
        ("log_decay", c_void_p), ("v_scale", c_void_p),
        ("q_scale", c_float),
        ("dq", c_void_p), ("dk", c_void_p), ("dv", c_void_p),
        ("dlog_decay", c_void_p), ("dv_scale", c_void_p),
        ("workspace", c_void_p), ("workspace_bytes", c_size_t),
    ]


class MlaParams(Structure):
    _fields_ = [
        ("dtype", c_int32),
        ("batch", c_int32), ("heads_q", c_int32), ("seqlen_kv", c_int32), ("dim", c_int32), ("dim_pe", c_int32),
        ("num_split", c_int32),
        ("q", c_void_p), ("q_stride_b", c_int64), ("q_stride_h", c_int64),
        ("q_pe", c_void_p), ("qpe_stride_b", c_int64), ("qpe_stride_h", c_int64),
        ("kv", c_void_p), ("kv_stride_b", c_int64), ("kv_stride_s", c_int64),
        ("k_pe", c_void_p), ("kpe_stride_b", c_int64), ("kpe_stride_s", c_int64),
        ("o", c_void_p), ("o_stride_b", c_int64), ("o_stride_h", c_int64),
        ("lse", c_void_p),
        ("scale", c_float),
        ("workspace", c_void_p), ("workspace_bytes", c_size_t),
        ("kv_seqlens", c_void_p),
        ("block_table", c_void_p), ("block_table_stride", c_int64), ("page_size", c_int32),
        ("tile_scheduler_metadata", c_void_p), ("num_splits", c_void_p), ("num_sm_parts", c_int32),
    ]


_lib = None


def load_library(path: str = LIB_PATH) -> ctypes.CDLL:
    """Loads the shared library (once).  Raises if it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(path):
        raise MetaAttentionError(
            -100, f"{path} not found: build it with `python -m metaattention_amd.build` (there is no CPU fallback)")
    lib = ctypes.CDLL(path)
    lib.ma_version.restype = c_int
    lib.ma_last_error.restype = c_char_p
    lib.ma_attn_fwd.argtypes = [POINTER(AttnParams), c_void_p]
    lib.ma_attn_fwd.restype = c_int
    lib.ma_attn_workspace_bytes.argtypes = [POINTER(AttnParams)]
    lib.ma_attn_workspace_bytes.restype = c_size_t
    lib.ma_attn_bwd.argtypes = [POINTER(AttnBwdParams), c_void_p]
    lib.ma_attn_bwd.restype = c_int
    lib.ma_attn_bwd_workspace_bytes.argtypes = [POINTER(AttnBwdParams)]
    lib.ma_attn_bwd_workspace_bytes.restype = c_size_t
    lib.ma_linear_workspace_bytes.argtypes = [POINTER(LinearParams)]
    lib.ma_linear_workspace_bytes.restype = c_size_t
    lib.ma_linear_fwd.argtypes = [POINTER(LinearParams), c_void_p]
    lib.ma_linear_fwd.restype = c_int
    lib.ma_linear_bwd_workspace_bytes.argtypes = [POINTER(LinearBwdParams)]
    lib.ma_linear_bwd_workspace_bytes.restype = c_size_t
    lib.ma_linear_bwd.argtypes = [POINTER(LinearBwdParams), c_void_p]
    lib.ma_linear_bwd.restype = c_int
    lib.ma_mla_choose_split.argtypes = [POINTER(MlaParams)]
    lib.ma_mla_choose_split.restype = c_int
    lib.ma_mla_workspace_bytes.argtypes = [POINTER(MlaParams)]
    lib.ma_mla_workspace_bytes.restype = c_size_t
    lib.ma_mla_decode.argtypes = [POINTER(MlaParams), c_void_p]
    lib.ma_mla_decode_noalloc.argtypes = [POINTER(MlaParams), c_void_p]
    lib.ma_mla_decode_noalloc.restype = c_int
    lib.ma_mla_noalloc_max_workspace.argtypes = []
    lib.ma_mla_noalloc_max_workspace.restype = c_size_t
    lib.ma_mla_num_sm_parts.argtypes = [c_int]
    lib.ma_mla_num_sm_parts.restype = c_int
    lib.ma_mla_get_metadata.argtypes = [c_void_p, c_int, c_int, c_void_p, c_void_p, c_void_p]
    lib.ma_mla_get_metadata.restype = c_int
    lib.ma_mla_decode.restype = c_int
    _lib = lib
    return lib


def _check(rc: int):
    if rc != 0:
        raise MetaAttentionError(rc, load_library().ma_last_error().decode())


def _dtype_code(dt: torch.dtype) -> int:
    if dt == torch.bfloat16:
        return MA_BF16
    if dt == torch.float16:
        return MA_FP16
    raise KeyError(dt)  # same failure mode as the reference's dtype map (attn_engine.py:234-237)


def _stream() -> int:
    return torch.cuda.current_stream().cuda_stream


def _require_gpu(*tensors):
    for t in tensors:
        if t is not None and not t.is_cuda:
            raise MetaAttentionError(-101, "tensors must live on the GPU (there is no CPU path)")


def attn_fwd(q, k, v, *, family: int, causal: bool, scale: float, bias: float = 0.0, bias_tensor=None,
             score_mask=None, out=None, row_scale=None, kv_seqlens=None, kv_block_mask=None, kv_block_size: int = 0,
             workspace=None, split_kv: bool = True, elem_mask=None, score_add=None, pos_slope_q=None, pos_slope_kv=None,
             softcap: float = 0.0, decay_gamma=None):
    """Parallel attention forward on BSHD tensors.  Returns ``out`` ([B,Sq,H,Dv]).  k and v may
    have fewer heads than q (grouped-query: query head h reads kv head h // (H // Hkv)).
    score_add: fp32 or q.dtype tensor broadcastable as [B|1, H|1, Sq|1, Skv|1] added to the scaled score;
    pos_slope_q / pos_slope_kv: fp32 [H], the score gets slope_q[h] * q_idx + slope_kv[h] * kv_idx;
    softcap > 0: softmax of softcap * tanh(x).
    decay_gamma: fp32 [H], for the retention family at 256 / 512 instead of score_mask: the multiplier is
    gamma[h]^(q - kv) below and on the diagonal, generated by the kernel."""
    _require_gpu(q, k, v, bias_tensor, score_mask, out, row_scale, kv_seqlens, kv_block_mask, score_add, pos_slope_q, pos_slope_kv)
    B, Sq, H, Dqk = q.shape
    Skv, Hkv, Dv = k.shape[1], k.shape[2], v.shape[-1]
    assert k.shape == (B, Skv, Hkv, Dqk) and v.shape == (B, Skv, Hkv, Dv) and H % Hkv == 0, "q/k/v shapes disagree"
    for t in (q, k, v):
        assert t.stride(-1) == 1, "last dimension must be contiguous"
    if out is None:
        out = torch.empty(B, Sq, H, Dv, dtype=q.dtype, device=q.device)
    p = AttnParams()
    p.family, p.dtype, p.mask = family, _dtype_code(q.dtype), MA_MASK_CAUSAL if causal else MA_MASK_NONE
    p.batch, p.heads, p.seqlen_q, p.seqlen_kv, p.dim_qk, p.dim_v = B, H, Sq, Skv, Dqk, Dv
    p.heads_kv = Hkv
    for name, t in (("q", q), ("k", k), ("v", v), ("o", out)):
        setattr(p, name, t.data_ptr())
        setattr(p, f"{name}_stride_b", t.stride(0))
        setattr(p, f"{name}_stride_s", t.stride(1))
        setattr(p, f"{name}_stride_h", t.stride(2))
    if row_scale is not None:
        assert row_scale.dtype == torch.float32 and row_scale.shape == (B, H, Sq) and row_scale.is_contiguous()
        p.row_scale = row_scale.data_ptr()
    p.scale, p.bias = float(scale), float(bias)
    if bias_tensor is not None:
        assert bias_tensor.dtype == torch.float32 and bias_tensor.numel() == 1
        p.bias_ptr = bias_tensor.data_ptr()
    if score_mask is not None:
        assert score_mask.dtype == q.dtype and score_mask.dim() == 4 and score_mask.stride(-1) == 1
        assert score_mask.shape[1:] == (H, Sq, Skv) and score_mask.shape[0] in (1, B)
        p.score_mask = score_mask.data_ptr()
        p.sm_stride_b = score_mask.stride(0) if score_mask.shape[0] > 1 else 0
        p.sm_stride_h, p.sm_stride_q = score_mask.stride(1), score_mask.stride(2)
    if kv_seqlens is not None:
        assert kv_seqlens.dtype == torch.int32 and kv_seqlens.shape == (B,) and kv_seqlens.is_contiguous()
        p.kv_seqlens = kv_seqlens.data_ptr()
    if kv_block_mask is not None:
        nblk = (Skv + kv_block_size - 1) // kv_block_size
        assert kv_block_mask.dtype in (torch.bool, torch.uint8) and kv_block_mask.stride(-1) == 1 and kv_block_mask.is_cuda
        p.kv_block_mask, p.kv_block_size = kv_block_mask.data_ptr(), int(kv_block_size)
        if kv_block_mask.dim() == 3:          # decode form: per (batch, kv head)
            assert kv_block_mask.shape == (B, Hkv, nblk)
            p.kbm_stride_b, p.kbm_stride_h = kv_block_mask.stride(0), kv_block_mask.stride(1)
        else:                                 # prefill form: per (batch | 1, query head | 1, block of 128 query rows)
            assert kv_block_mask.shape[2:] == ((Sq + 127) // 128, nblk) and kv_block_mask.shape[0] in (1, B) and kv_block_mask.shape[1] in (1, H)
            p.kbm_stride_b = kv_block_mask.stride(0) if kv_block_mask.shape[0] > 1 else 0
            p.kbm_stride_h = kv_block_mask.stride(1) if kv_block_mask.shape[1] > 1 else 0
            p.kbm_stride_q, p.kbm_per_query_head = kv_block_mask.stride(2), 1
    if elem_mask is not None:
        assert elem_mask.dtype in (torch.bool, torch.uint8) and elem_mask.dim() == 4 and elem_mask.shape[2:] == (Sq, Skv)
        assert elem_mask.shape[0] in (1, B) and elem_mask.shape[1] in (1, H) and elem_mask.stride(-1) == 1 and elem_mask.is_cuda
        p.elem_mask = elem_mask.data_ptr()
        p.em_stride_b = elem_mask.stride(0) if elem_mask.shape[0] > 1 else 0
        p.em_stride_h = elem_mask.stride(1) if elem_mask.shape[1] > 1 else 0
        p.em_stride_q = elem_mask.stride(2)
    if score_add is not None:
        assert score_add.dim() == 4 and score_add.dtype in (torch.float32, q.dtype)
        for ax, full in enumerate((B, H, Sq, Skv)):
            assert score_add.shape[ax] in (1, full), f"score_add {tuple(score_add.shape)} does not broadcast to {(B, H, Sq, Skv)}"
        st = [score_add.stride(ax) if score_add.shape[ax] > 1 else 0 for ax in range(4)]
        p.score_add, p.score_add_fp32 = score_add.data_ptr(), int(score_add.dtype == torch.float32)
        p.sa_stride_b, p.sa_stride_h, p.sa_stride_q, p.sa_stride_kv = st
    for name, t in (("pos_slope_q", pos_slope_q), ("pos_slope_kv", pos_slope_kv)):
        if t is not None:
            assert t.dtype == torch.float32 and t.shape == (H,) and t.is_contiguous()
            setattr(p, name, t.data_ptr())
    p.softcap = float(softcap)
    if decay_gamma is not None:
        assert decay_gamma.dtype == torch.float32 and decay_gamma.shape == (H,) and decay_gamma.is_contiguous() and decay_gamma.is_cuda
        p.decay_gamma = decay_gamma.data_ptr()
    lib = load_library()
    if split_kv:
        need = lib.ma_attn_workspace_bytes(ctypes.byref(p))
        if need:
            if workspace is None:
                workspace = torch.empty(need, dtype=torch.uint8, device=q.device)
            assert workspace.numel() * workspace.element_size() >= need
            p.workspace, p.workspace_bytes = workspace.data_ptr(), workspace.numel() * workspace.element_size()
    _check(lib.ma_attn_fwd(ctypes.byref(p), _stream()))
    return out


def attn_bwd(q, k, v, o, dout, lse, *, family: int, causal: bool, scale: float, bias: float = 0.0, bias_tensor=None,
             elem_mask=None, elem_mask_t=None, kv_block_mask=None, q_block_mask=None, score_mask=None, score_mask_t=None,
             score_add=None, pos_slope_q=None, pos_slope_kv=None, softcap: float = 0.0):
    """Gradients (dq, dk, dv) of the parallel attention forward on BSHD tensors.  ``o`` and ``lse``
    (fp32 [B,H,Sq]) are the forward pass's output and row scale (softmax and retention; None otherwise),
    ``dout`` the gradient of ``o``.  The retention family takes the forward's multiplier tensor ``score_mask``
    [1|B, H, Sq, Skv] and its transpose ``score_mask_t`` [1|B, H, Skv, Sq] in the tensor dtype, and treats the
    row scale as a constant, as the reference's OnlineRetention.backward does.  ``elem_mask`` (the forward pass's keep mask, [1|B, 1|H, Sq, Skv]) comes with
    its transpose ``elem_mask_t`` [1|B, 1|H, Skv, Sq]; both with rows at 4-byte aligned addresses.  Optional tile masks
    for skipping: ``kv_block_mask`` [1|B, 1|H, ceil(Sq/128), ceil(Skv/32)] and ``q_block_mask`` [1|B, 1|H, ceil(Skv/128),
    ceil(Sq/32)] (a tile is kept when any of its elements is).  ``score_add``, ``pos_slope_q`` / ``pos_slope_kv`` and
    ``softcap`` (softmax, sigmoid and relu families; softcap with softmax only) are the forward pass's additive score terms and soft-capping, given again unchanged; they
    receive no gradients of their own."""
    _require_gpu(q, k, v, o, dout, lse, bias_tensor, elem_mask, elem_mask_t, kv_block_mask, q_block_mask, score_mask, score_mask_t,
                 score_add, pos_slope_q, pos_slope_kv)
    B, Sq, H, Dqk = q.shape
    Skv, Hkv, Dv = k.shape[1], k.shape[2], v.shape[-1]
    assert k.shape == (B, Skv, Hkv, Dqk) and v.shape == (B, Skv, Hkv, Dv) and dout.shape == (B, Sq, H, Dv) and H % Hkv == 0
    dout = dout if dout.stride(-1) == 1 else dout.contiguous()
    dq, dk, dv = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)
    p = AttnBwdParams()
    p.family, p.dtype, p.mask = family, _dtype_code(q.dtype), MA_MASK_CAUSAL if causal else MA_MASK_NONE
    p.batch, p.heads, p.heads_kv, p.seqlen_q, p.seqlen_kv, p.dim_qk, p.dim_v = B, H, Hkv, Sq, Skv, Dqk, Dv
    for name, prefix, t in (("q", "q", q), ("k", "k", k), ("v", "v", v), ("o", "o", o), ("dout", "do", dout), ("dq", "dq", dq),
                            ("dk", "dk", dk), ("dv", "dv", dv)):
        if t is None:
            continue
        assert t.stride(-1) == 1 and t.dtype == q.dtype, "last dimension must be contiguous, one dtype"
        setattr(p, name, t.data_ptr())
        setattr(p, f"{prefix}_stride_b", t.stride(0))
        setattr(p, f"{prefix}_stride_s", t.stride(1))
        setattr(p, f"{prefix}_stride_h", t.stride(2))
    if lse is not None:
        assert lse.dtype == torch.float32 and lse.shape == (B, H, Sq) and lse.is_contiguous()
        p.lse = lse.data_ptr()
    p.scale, p.bias = float(scale), float(bias)
    if bias_tensor is not None:
        assert bias_tensor.dtype == torch.float32 and bias_tensor.numel() == 1
        p.bias_ptr = bias_tensor.data_ptr()
    if elem_mask is not None or elem_mask_t is not None:
        assert elem_mask is not None and elem_mask_t is not None, "elem_mask and elem_mask_t go together"
        for t, rows, cols, pre, last in ((elem_mask, Sq, Skv, "em", "q"), (elem_mask_t, Skv, Sq, "emt", "k")):
            assert t.dtype in (torch.bool, torch.uint8) and t.dim() == 4 and t.shape[2:] == (rows, cols) and t.stride(-1) == 1
            assert t.shape[0] in (1, B) and t.shape[1] in (1, H)
            setattr(p, "elem_mask" if pre == "em" else "elem_mask_t", t.data_ptr())
            setattr(p, f"{pre}_stride_b", t.stride(0) if t.shape[0] > 1 else 0)
            setattr(p, f"{pre}_stride_h", t.stride(1) if t.shape[1] > 1 else 0)
            setattr(p, f"{pre}_stride_{last}", t.stride(2))
    if kv_block_mask is not None or q_block_mask is not None:
        assert kv_block_mask is not None and q_block_mask is not None, "kv_block_mask and q_block_mask go together"
        for t, shape, pre, last in ((kv_block_mask, ((Sq + 127) // 128, (Skv + 31) // 32), "kbm", "q"),
                                    (q_block_mask, ((Skv + 127) // 128, (Sq + 31) // 32), "qbm", "k")):
            assert t.dtype in (torch.bool, torch.uint8) and t.dim() == 4 and t.shape[2:] == shape and t.stride(-1) == 1
            assert t.shape[0] in (1, B) and t.shape[1] in (1, H)
            setattr(p, "kv_block_mask" if pre == "kbm" else "q_block_mask", t.data_ptr())
            setattr(p, f"{pre}_stride_b", t.stride(0) if t.shape[0] > 1 else 0)
            setattr(p, f"{pre}_stride_h", t.stride(1) if t.shape[1] > 1 else 0)
            setattr(p, f"{pre}_stride_{last}", t.stride(2))
    if score_mask is not None or score_mask_t is not None:
        assert score_mask is not None and score_mask_t is not None, "score_mask and score_mask_t go together"
        for t, rows, cols, pre, last in ((score_mask, Sq, Skv, "sm", "q"), (score_mask_t, Skv, Sq, "smt", "k")):
            assert t.dtype == q.dtype and t.dim() == 4 and t.shape[1:] == (H, rows, cols) and t.shape[0] in (1, B) and t.stride(-1) == 1
            setattr(p, "score_mask" if pre == "sm" else "score_mask_t", t.data_ptr())
            setattr(p, f"{pre}_stride_b", t.stride(0) if t.shape[0] > 1 else 0)
            setattr(p, f"{pre}_stride_h", t.stride(1))
            setattr(p, f"{pre}_stride_{last}", t.stride(2))
    if score_add is not None:
        assert score_add.dim() == 4 and score_add.dtype in (torch.float32, q.dtype)
        for ax, full in enumerate((B, H, Sq, Skv)):
            assert score_add.shape[ax] in (1, full), f"score_add {tuple(score_add.shape)} does not broadcast to {(B, H, Sq, Skv)}"
        st = [score_add.stride(ax) if score_add.shape[ax] > 1 else 0 for ax in range(4)]
        p.score_add, p.score_add_fp32 = score_add.data_ptr(), int(score_add.dtype == torch.float32)
        p.sa_stride_b, p.sa_stride_h, p.sa_stride_q, p.sa_stride_kv = st
    for name, t in (("pos_slope_q", pos_slope_q), ("pos_slope_kv", pos_slope_kv)):
        if t is not None:
            assert t.dtype == torch.float32 and t.numel() == H and t.is_contiguous()
            setattr(p, name, t.data_ptr())
    p.softcap = float(softcap)
    lib = load_library()
    need = lib.ma_attn_bwd_workspace_bytes(ctypes.byref(p))
    if need:
        ws = torch.empty(need, dtype=torch.uint8, device=q.device)
        p.workspace, p.workspace_bytes = ws.data_ptr(), need
    _check(lib.ma_attn_bwd(ctypes.byref(p), _stream()))
    return dq, dk, dv


def mla_decode(q, q_pe, kv, k_pe, *, scale: float, num_split: int = 0, out=None, lse=None, workspace=None, kv_seqlens=None,
               no_alloc: bool = False):
    """Absorbed MLA decode.  q [B,1,Hq,D], q_pe [B,1,Hq,Dpe], kv [B,Skv,1,D],
    k_pe [B,Skv,1,Dpe] (the reference operator's layouts) -> [B,1,Hq,D].
    no_alloc=True goes through ma_mla_decode_noalloc: the partial results of the kv splits live in the library's own
    scratch array instead of a workspace tensor (``out`` must then be given, so that this call allocates nothing)."""
    _require_gpu(q, q_pe, kv, k_pe, out, lse, workspace)
    B, one, Hq, D = q.shape
    Skv, Dpe = kv.shape[1], q_pe.shape[-1]
    assert one == 1 and kv.shape[2] == 1 and k_pe.shape == (B, Skv, 1, Dpe) and q_pe.shape == (B, 1, Hq, Dpe)
    for t in (q, q_pe, kv, k_pe):
        assert t.stride(-1) == 1, "last dimension must be contiguous"
    if out is None:
        assert not no_alloc, "no_alloc=True needs the output tensor"
        out = torch.empty(B, 1, Hq, D, dtype=q.dtype, device=q.device)
    p = MlaParams()
    p.dtype = _dtype_code(q.dtype)
    p.batch, p.heads_q, p.seqlen_kv, p.dim, p.dim_pe, p.num_split = B, Hq, Skv, D, Dpe, num_split
    p.q, p.q_stride_b, p.q_stride_h = q.data_ptr(), q.stride(0), q.stride(2)
    p.q_pe, p.qpe_stride_b, p.qpe_stride_h = q_pe.data_ptr(), q_pe.stride(0), q_pe.stride(2)
    p.kv, p.kv_stride_b, p.kv_stride_s = kv.data_ptr(), kv.stride(0), kv.stride(1)
    p.k_pe, p.kpe_stride_b, p.kpe_stride_s = k_pe.data_ptr(), k_pe.stride(0), k_pe.stride(1)
    p.o, p.o_stride_b, p.o_stride_h = out.data_ptr(), out.stride(0), out.stride(2)
    if lse is not None:
        assert lse.dtype == torch.float32 and lse.shape == (B, Hq) and lse.is_contiguous()
        p.lse = lse.data_ptr()
    p.scale = float(scale)
    if kv_seqlens is not None:
        assert kv_seqlens.dtype == torch.int32 and kv_seqlens.shape == (B,) and kv_seqlens.is_contiguous() and kv_seqlens.is_cuda
        p.kv_seqlens = kv_seqlens.data_ptr()
    lib = load_library()
    if no_alloc:
        _check(lib.ma_mla_decode_noalloc(ctypes.byref(p), _stream()))
        return out
    need = lib.ma_mla_workspace_bytes(ctypes.byref(p))
    if need:
        if workspace is None:
            workspace = torch.empty(need, dtype=torch.uint8, device=q.device)
        assert workspace.numel() * workspace.element_size() >= need
        p.workspace, p.workspace_bytes = workspace.data_ptr(), workspace.numel() * workspace.element_size()
    _check(lib.ma_mla_decode(ctypes.byref(p), _stream()))
    return out


def get_mla_metadata(cache_seqlens, num_heads_per_head_k: int, num_heads_k: int, num_sm_parts: int = 0):
    """get_mla_metadata of the paged MLA interface (cute_template_kvshared/flash_mla_interface.py:57-72): the work plan
    for a ragged batch, computed on the device from cache_seqlens (int32 [B]) by the greedy scheme of
    kernels/get_mla_metadata.cu:8-75.  Returns (tile_scheduler_metadata int32 [num_sm_parts, 8], num_splits int32 [B + 1]);
    flash_mla_with_kvcache hands every workgroup the run of (batch entry, token range) pieces its part names.
    num_sm_parts defaults to one part per CU and block of 128 query heads."""
    _require_gpu(cache_seqlens)
    assert num_heads_k == 1, "one latent kv head"
    lib = load_library()
    seqlens = cache_seqlens.to(torch.int32).contiguous()
    B = seqlens.shape[0]
    parts = int(num_sm_parts) if num_sm_parts else lib.ma_mla_num_sm_parts(int(num_heads_per_head_k))
    meta = torch.empty(parts, 8, dtype=torch.int32, device=seqlens.device)
    splits = torch.empty(B + 1, dtype=torch.int32, device=seqlens.device)
    _check(lib.ma_mla_get_metadata(seqlens.data_ptr(), B, parts, meta.data_ptr(), splits.data_ptr(), _stream()))
    return meta, splits


def flash_mla_with_kvcache(q, k_cache, block_table, cache_seqlens, head_dim_v: int, tile_scheduler_metadata=None, num_splits=None,
                           softmax_scale=None, causal: bool = False):
    """Paged absorbed-MLA decode with the signature of flash_mla_with_kvcache
    (cute_template_kvshared/flash_mla_interface.py:75-115): q [B,1,Hq,576], k_cache [pages, page_size, 1, 576]
    (latent 512 + rope 64 in one row), block_table int32 [B, pages per sequence], cache_seqlens int32 [B]
    -> (out [B,1,Hq,512], softmax_lse fp32 [B,Hq,1], natural log).  One query token, so `causal` changes nothing."""
    _require_gpu(q, k_cache, block_table, cache_seqlens)
    B, Sq, Hq, Dfull = q.shape
    assert Sq == 1 and k_cache.shape[2] == 1 and k_cache.shape[3] == Dfull and head_dim_v < Dfull, "one query token, one latent kv head"
    page = k_cache.shape[1]
    assert block_table.dtype == torch.int32 and block_table.shape[0] == B and block_table.stride(1) == 1
    assert q.stride(-1) == 1 and k_cache.is_contiguous()
    D, Dpe = head_dim_v, Dfull - head_dim_v
    scale = Dfull ** -0.5 if softmax_scale is None else softmax_scale
    out = torch.empty(B, 1, Hq, D, dtype=q.dtype, device=q.device)
    lse = torch.empty(B, Hq, dtype=torch.float32, device=q.device)
    seqlens = cache_seqlens.to(torch.int32).contiguous()
    p = MlaParams()
    p.dtype = _dtype_code(q.dtype)
    p.batch, p.heads_q, p.seqlen_kv, p.dim, p.dim_pe, p.num_split = B, Hq, block_table.shape[1] * page, D, Dpe, 0
    esz = q.element_size()
    p.q, p.q_stride_b, p.q_stride_h = q.data_ptr(), q.stride(0), q.stride(2)
    p.q_pe, p.qpe_stride_b, p.qpe_stride_h = q.data_ptr() + D * esz, q.stride(0), q.stride(2)
    p.kv, p.kv_stride_b, p.kv_stride_s = k_cache.data_ptr(), 0, Dfull
    p.k_pe, p.kpe_stride_b, p.kpe_stride_s = k_cache.data_ptr() + D * esz, 0, Dfull
    p.o, p.o_stride_b, p.o_stride_h = out.data_ptr(), out.stride(0), out.stride(2)
    p.lse, p.scale = lse.data_ptr(), float(scale)
    p.kv_seqlens = seqlens.data_ptr()
    p.block_table, p.block_table_stride, p.page_size = block_table.data_ptr(), block_table.stride(0), page
    if tile_scheduler_metadata is not None and tile_scheduler_metadata.dim() == 2 and tile_scheduler_metadata.shape[1] == 8:
        # the plan of get_mla_metadata: every workgroup walks its part's pieces
        assert num_splits is not None and num_splits.shape == (B + 1,), "num_splits of get_mla_metadata goes with its metadata"
        assert tile_scheduler_metadata.dtype == torch.int32 and num_splits.dtype == torch.int32
        assert tile_scheduler_metadata.is_contiguous() and num_splits.is_contiguous()
        _require_gpu(tile_scheduler_metadata, num_splits)
        p.tile_scheduler_metadata, p.num_splits = tile_scheduler_metadata.data_ptr(), num_splits.data_ptr()
        p.num_sm_parts = tile_scheduler_metadata.shape[0]
    lib = load_library()
    need = lib.ma_mla_workspace_bytes(ctypes.byref(p))
    if need:
        workspace = torch.empty(need, dtype=torch.uint8, device=q.device)
        p.workspace, p.workspace_bytes = workspace.data_ptr(), need
    _check(lib.ma_mla_decode(ctypes.byref(p), _stream()))
    return out, lse.view(B, Hq, 1)


def mla_workspace_bytes(B, Hq, Skv, D=512, Dpe=64, num_split=0) -> int:
    p = MlaParams()
    p.batch, p.heads_q, p.seqlen_kv, p.dim, p.dim_pe, p.num_split = B, Hq, Skv, D, Dpe, num_split
    return load_library().ma_mla_workspace_bytes(ctypes.byref(p))


def linear_fwd(q, k, v, log_decay, *, q_scale: float = 1.0, v_scale=None, chunk=None, out=None, segments: int = 0,
               workspace=None, out_fp32: bool = False):
    """Chunked linear attention forward on BHSD tensors: q [B,Hq,T,Dk], k [B,Hk,T,Dk],
    v [B,H,T,Dv] (bf16, contiguous), log_decay fp32 [B,H,T], optional per-token value
    scale [B,H,T].  ``chunk`` is accepted for API compatibility; the result does not
    depend on it and the kernel uses its own chunking.  ``segments``: 0 lets the library
    decide whether to cut the sequence into segments that run side by side (it does when
    batch x heads is small), 1 forces the single pass, n allows up to n segments; the
    workspace that needs is allocated here unless one is passed."""
    _require_gpu(q, k, v, log_decay, v_scale, out, workspace)
    B, H, T, Dv = v.shape
    Hq, Hk, Dk = q.shape[1], k.shape[1], q.shape[-1]
    assert q.shape == (B, Hq, T, Dk) and k.shape == (B, Hk, T, Dk), "q/k/v shapes disagree"
    assert log_decay.shape == (B, H, T), "log_decay must be [B,H,T]"
    q, k, v = q.contiguous(), k.contiguous(), v.contiguous()
    log_decay = log_decay.to(torch.float32).contiguous()
    if v_scale is not None:
        assert v_scale.shape == (B, H, T)
        v_scale = v_scale.to(torch.float32).contiguous()
    if out is None:
        out = torch.empty(B, H, T, Dv, dtype=torch.float32 if out_fp32 else v.dtype, device=v.device)
    assert out.dtype == (torch.float32 if out_fp32 else v.dtype) and out.is_contiguous()
    p = LinearParams()
    p.out_fp32 = int(out_fp32)
    p.dtype = _dtype_code(v.dtype)
    p.batch, p.heads, p.heads_q, p.heads_k, p.seqlen, p.dim_k, p.dim_v = B, H, Hq, Hk, T, Dk, Dv
    p.chunk = int(chunk or 0)
    p.q, p.k, p.v, p.o = q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr()
    p.log_decay = log_decay.data_ptr()
    p.v_scale = v_scale.data_ptr() if v_scale is not None else None
    p.q_scale = float(q_scale)
    p.segments = int(segments)
    lib = load_library()
    need = lib.ma_linear_workspace_bytes(ctypes.byref(p))
    if need > 0:
        if workspace is None:
            workspace = torch.empty(need, dtype=torch.uint8, device=v.device)
        assert workspace.numel() * workspace.element_size() >= need
        p.workspace, p.workspace_bytes = workspace.data_ptr(), workspace.numel() * workspace.element_size()
    _check(lib.ma_linear_fwd(ctypes.byref(p), _stream()))
    return out


def linear_bwd(q, k, v, log_decay, dout, *, q_scale: float = 1.0, v_scale=None, workspace=None):
    """Gradients of linear_fwd with respect to q, k, v, log_decay and v_scale (None when no v_scale):
    (dq, dk, dv, dlog_decay, dv_scale) with dq, dk, dv in the tensors' dtype (the gradients of heads that share a
    q / k head summed, as LinearAttention.backward does, linear_tl.py:1300-1303) and the two per-token gradients in
    fp32 [B,H,T].  One call of ma_linear_bwd; the workspace it needs is allocated here unless one is passed."""
    _require_gpu(q, k, v, log_decay, dout, v_scale, workspace)
    B, H, T, Dv = v.shape
    Hq, Hk, Dk = q.shape[1], k.shape[1], q.shape[-1]
    assert q.shape == (B, Hq, T, Dk) and k.shape == (B, Hk, T, Dk) and dout.shape == v.shape, "q/k/v/dout shapes disagree"
    assert log_decay.shape == (B, H, T), "log_decay must be [B,H,T]"
    q, k, v = q.contiguous(), k.contiguous(), v.contiguous()
    dout = dout.to(v.dtype).contiguous()
    g = log_decay.to(torch.float32).contiguous()
    vs = None
    if v_scale is not None:
        assert v_scale.shape == (B, H, T)
        vs = v_scale.to(torch.float32).contiguous()
    dq, dk, dv = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)
    dld = torch.empty(B, H, T, dtype=torch.float32, device=v.device)
    dvs = torch.empty(B, H, T, dtype=torch.float32, device=v.device) if vs is not None else None
    p = LinearBwdParams()
    p.dtype = _dtype_code(v.dtype)
    p.batch, p.heads, p.heads_q, p.heads_k, p.seqlen, p.dim_k, p.dim_v = B, H, Hq, Hk, T, Dk, Dv
    p.q, p.k, p.v, p.dout = q.data_ptr(), k.data_ptr(), v.data_ptr(), dout.data_ptr()
    p.log_decay = g.data_ptr()
    p.v_scale = vs.data_ptr() if vs is not None else None
    p.q_scale = float(q_scale)
    p.dq, p.dk, p.dv, p.dlog_decay = dq.data_ptr(), dk.data_ptr(), dv.data_ptr(), dld.data_ptr()
    p.dv_scale = dvs.data_ptr() if dvs is not None else None
    lib = load_library()
    need = lib.ma_linear_bwd_workspace_bytes(ctypes.byref(p))
    if need > 0:
        if workspace is None:
            workspace = torch.empty(need, dtype=torch.uint8, device=v.device)
        p.workspace, p.workspace_bytes = workspace.data_ptr(), workspace.numel() * workspace.element_size()   # (a small one is refused by the library)
    _check(lib.ma_linear_bwd(ctypes.byref(p), _stream()))
    return dq, dk, dv, dld, dvs


def linear_workspace_bytes(B, H, Hq, Hk, T, Dk, Dv, segments: int = 0) -> int:
    p = LinearParams()
    p.dtype, p.batch, p.heads, p.heads_q, p.heads_k, p.seqlen, p.dim_k, p.dim_v, p.segments = MA_BF16, B, H, Hq, Hk, T, Dk, Dv, segments
    return load_library().ma_linear_workspace_bytes(ctypes.byref(p))
