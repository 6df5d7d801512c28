"""``LinearAttentionEngine``: chunked linear / stateful attention operator
(attention_engine/attn_engine/linear_attn_engine.py:11-65) on the gfx950
kernel library.

``mod(q, k, v, decay, *custom)`` with q [B,Hq,T,Dk], k [B,Hk,T,Dk],
v [B,H,T,Dv] (bf16, BHSD), decay fp32 [B,H,T] and the custom tensors in
``CustomIO`` order returns o [B,H,T,Dv]:

    o_t = q_mod(q_t) . sum_{s<=t} exp(G_t - G_s) k_mod(k_s)^T v_mod(v_s),   G = cumsum(decay_mod(decay))
"""
from __future__ import annotations

import torch

from core.canonical import canonicalize_linear_mods
from core.eager import evaluate, custom_tensor_view
from core.transform.core import CustomIO


class _LinearAttention(torch.autograd.Function):
    """Forward + backward of the chunked operator on (q, k, v, log decay, value scale), as LinearAttention
    of tl_template/linear/linear_tl.py:1240-1340; the mods around it (decay_mod, the tensors behind v_mod)
    are ordinary PyTorch operations, so autograd carries the gradients on to decay, A, dt."""

    @staticmethod
    def forward(ctx, q, k, v, g, v_scale, q_scale, chunk):
        from hip_backend import linear_fwd
        ctx.q_scale = q_scale
        ctx.has_vs = v_scale is not None
        ctx.save_for_backward(q, k, v, g, *([v_scale] if v_scale is not None else []))
        return linear_fwd(q, k, v, g, q_scale=q_scale, v_scale=v_scale, chunk=chunk)

    @staticmethod
    def backward(ctx, dout):
        from hip_backend import linear_bwd
        q, k, v, g, *rest = ctx.saved_tensors
        vs = rest[0] if ctx.has_vs else None
        dq, dk, dv, dg, dvs = linear_bwd(q, k, v, g, dout, q_scale=ctx.q_scale, v_scale=vs)
        if dvs is not None:
            dvs = dvs.to(vs.dtype)
        return dq, dk, dv, dg.to(g.dtype), dvs, None, None


class LinearAttentionEngine:
    def __init__(self, qkv_meta, q_mod=None, k_mod=None, v_mod=None, decay_mod=None, custom_io=None,
                 tune=False, tune_filename="tune_result", tune_bwd=False, chunk_size=None):
        # tune* select the reference's tile search; fixed CDNA4 tiles here.
        self.custom_io = custom_io if custom_io is not None else CustomIO()
        self.names = list(self.custom_io.input_tensors)
        self.plan = canonicalize_linear_mods(q_mod, k_mod, v_mod, decay_mod, self.custom_io)
        self.dtype = qkv_meta[0].dtype
        if self.dtype != torch.bfloat16:
            raise KeyError(self.dtype)    # the linear kernels are bf16 only (linear_tl.py:129,299)
        self.meta = dict(B=qkv_meta[0].shape[0], Hq=qkv_meta[0].shape[1], Hk=qkv_meta[1].shape[1], H=qkv_meta[2].shape[1],
                         T=qkv_meta[0].shape[2], Dk=qkv_meta[0].shape[3], Dv=qkv_meta[2].shape[3])
        self.chunk_size = chunk_size
        self.tl_code = ""
        self.attention = self._call

    def _log_decay(self, decay, given):
        """decay_mod evaluated on the [B,H,T] fp32 decay input.  Like the
        reference, which emits this mod as eager PyTorch (linear_tl.py:1250-1256),
        it is a tiny element-wise prologue on the GPU."""
        plan = self.plan
        if plan.decay_sym is None:
            return decay
        if plan.decay_kind == "log":
            return torch.log(decay)
        if plan.decay_kind == "mul_head":
            return decay * given[plan.decay_head_tensor].to(torch.float32).reshape(1, -1, 1)
        env = {id(plan.decay_in): decay}
        for n, sym in self.custom_io.input_tensors.items():
            t = given[n].to(torch.float32)
            view = custom_tensor_view(t, sym.shape_idx)           # [B|1, H|1, T|1, 1]
            env[id(sym)] = view.reshape(view.shape[:3])
        (out,) = evaluate([plan.decay_sym], env, decay)
        return out.expand_as(decay).contiguous()

    def _call(self, q, k, v, decay, *custom):
        from hip_backend import linear_fwd
        if len(custom) != len(self.names):
            raise TypeError(f"expected {len(self.names)} custom tensor(s) {self.names} after q, k, v, decay; got {len(custom)}")
        given = dict(zip(self.names, custom))
        g = self._log_decay(decay.to(torch.float32), given)
        v_scale = given[self.plan.v_scale_tensor] if self.plan.v_scale_tensor else None

        if any(t is not None and t.requires_grad for t in (q, k, v, g, v_scale)):
            return _LinearAttention.apply(q, k, v, g, v_scale, self.plan.q_scale, self.chunk_size)
        return linear_fwd(q, k, v, g, q_scale=self.plan.q_scale, v_scale=v_scale, chunk=self.chunk_size)

    def __call__(self, *args, **kargs):
        return self.attention(*args, **kargs)
