#!/usr/bin/env python3
"""Benchmark of the attention forward hot path on one MI355X.

A step is one forward pass of the headline workload: causal softmax MHA, bf16
in / fp32 accumulate, B=8 H=32 S=4096 D=128 (synthetic N(0,1) inputs already
resident in HBM).  Prints ONE JSON line; `value` is algorithmic TFLOP/s
(causal counted at one half: 0.5 * 4 * B*H*S^2*D FLOP per pass).  The same line
carries the roofline of the dominant kernel, a CPU baseline (the oracle's
restated PyTorch reference timed on this box's host cores over a bounded
sample of the same workload) and, under "other_workloads", the remaining
benchmark configurations, each with its own roofline fraction (and, for C3, C4 and C5, the oracle timed on the host
cores over a bounded sample as "cpu_baseline"):

  c2_sigmoid_causal   same shape, sigmoid(q.k*scale - log S) row function
  c2_softmax_causal_operator  the headline workload through the operator AttentionEngine returns (with its allocations)
  c2_softmax_causal_bwd  backward of the headline workload (dq, dk, dv)
  c3_retnet_chunked   RetNet retention, chunked operator, B8 H16 S2048 Dqk256 Dv512
  c3_retnet_parallel  same shape, normalised parallel operator with a [1,H,S,S] decay mask
  c3_retnet_parallel_operator  the same through the operator AttentionEngine returns, mod(q, k, v, mask): it recognises the decay mask
  c3_retnet_parallel_generated_mask  the same operator told the mask is gamma_h^(i-j) (decay_gamma): no mask tensor is read
  c3_retnet_parallel_bwd  backward of that operator (dq, dk, dv; the row scale held constant, as the reference defines it)
  c4_mamba2_ssd       Mamba2 SSD, B8 H64 S2048 P64 N128, one B/C group
  c3_retnet_chunked_operator / c4_mamba2_ssd_operator / c5_mla_decode_operator  those three through the operators the engines return
  c5_mla_decode       absorbed MLA decode, B64 Hq128 KV4096 d512+64 (HBM bound)
  gqa_decode          grouped-query softmax decode, B64 H32 Hkv8 KV4096 D128 (HBM bound)
  reference_shapes    the MLA / RetNet / Mamba2 shapes whose kernel latencies the reference's tuned_config files record
  reference_benchmark_shapes  causal softmax at Dqk 192 / Dv 128 and ReLU attention at 64 / 64 as in testing/benchmark_mi250.py
"""
from __future__ import annotations

import argparse
import json
import math
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "metaattention_amd"))

PEAK_BF16_TFLOPS = 2500.0   # MI355X dense bf16 MFMA
PEAK_HBM_GBS = 8000.0       # MI355X HBM3E
# HBM bytes per launch of the headline kernel, from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE scaled by a 1 GiB copy: the
# profile summary of that kernel holds the figure in a line "hbm_traffic_bytes_per_launch[<kernel>]: <bytes>"
ATTN_FWD_PROFILE = os.path.join(ROOT, "profiles", "attn_fwd_kernel_c2_softmax_sigmoid.md")
ATTN_FWD_KERNEL = "ma::attn_fwd_kernel<bf16, 128, 128, 0, true>"   # (element type, Dqk, Dv, family 0 = softmax, causal)


def profiled_traffic(path, kernel):
    """(bytes per launch, file it was read from) from a profile summary, or (None, None)."""
    try:
        for ln in open(path):
            if ln.startswith("hbm_traffic_bytes_per_launch[" + kernel + "]:"):
                return float(ln.split(":", 3)[-1].strip()), os.path.relpath(path, ROOT)
    except OSError:
        pass
    return None, None


# The GPU's clocks take tens of milliseconds of load to settle after idle: measured on these boxes, a workload timed right
# after 5 warm-up launches runs 5 % (1.1 ms kernel) to 20 % (0.15 ms kernel) slower than the same workload a moment later.
# Every timing below therefore first keeps the device busy with the workload itself for RAMP_MS (--ramp-ms), then does the
# `warmup` launches, then times `steps` launches.
RAMP_MS = 80.0


def time_gpu(fn, steps, warmup, flush=None):
    """Average milliseconds per call over `steps` calls, HIP events on the launch stream.
    With `flush`, that callable runs before every call (it replaces what the caches hold) and each
    call is timed on its own (for the HBM-bound workloads)."""
    import torch
    t0 = time.perf_counter()
    while (time.perf_counter() - t0) * 1e3 < RAMP_MS:
        for _ in range(4):
            fn()
        torch.cuda.synchronize()
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    if flush is None:
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(steps):
            fn()
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) / steps
    total = 0.0
    for _ in range(steps):
        flush()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        fn()
        e1.record()
        torch.cuda.synchronize()
        total += e0.elapsed_time(e1)
    return total / steps


COLD_NOTE = ("ms / frac_of_hbm_peak_clean_read: 1 GiB of other data is READ through the caches before every timed call, so the call "
             "starts with cold caches that hold clean lines; ms_after_cache_overwrite / frac_of_hbm_peak: the same with that buffer "
             "WRITTEN instead -- the timed call then also pays for the write-back of the buffer's dirty lines (L2 and the "
             "last-level cache); ms_without_cache_flush: calls back to back")


def _junk():
    """1 GiB of int32 ones: more than L2 and the 256 MB last-level cache together."""
    import torch
    return torch.ones(2 ** 28, dtype=torch.int32, device="cuda")


def _hbm_entry(ms_clean, ms_dirty, ms_warm, nbytes):
    """An HBM-bound workload timed call by call in three cache states.  `frac_of_hbm_peak` is the figure after the
    OVERWRITING flush (a 1 GiB buffer written before every timed call: caches hold none of the workload, and the call also
    pays for the write-back of that buffer's dirty lines); `frac_of_hbm_peak_clean_read` after the same buffer was READ
    (cold caches holding clean lines: what a decode step meets in a serving loop); both against 8 TB/s."""
    gbs_dirty, gbs_clean = nbytes / ms_dirty / 1e6, nbytes / ms_clean / 1e6
    return dict(ms=round(ms_clean, 4), ms_after_cache_overwrite=round(ms_dirty, 4), ms_without_cache_flush=round(ms_warm, 4),
                gb_per_s=round(gbs_dirty, 1), frac_of_hbm_peak=round(gbs_dirty / PEAK_HBM_GBS, 4),
                gb_per_s_clean_read=round(gbs_clean, 1), frac_of_hbm_peak_clean_read=round(gbs_clean / PEAK_HBM_GBS, 4),
                algorithmic_bytes=nbytes)


def _mfma_entry(ms, flops, note=None, **extra):
    tf = flops / ms / 1e9
    d = dict(ms=round(ms, 4), tflops=round(tf, 1), frac_of_bf16_peak=round(tf / PEAK_BF16_TFLOPS, 4), algorithmic_flops=flops)
    if note:
        d["flop_convention"] = note
    d.update(extra)
    return d


def bench_softmax(steps, warmup, family="softmax", B=8, S=4096, causal=True):
    import torch
    from metaattention_amd import hip_backend as hb
    H, D = 32, 128
    g = torch.Generator(device="cuda").manual_seed(0)
    q, k, v = (torch.randn(B, S, H, D, device="cuda", dtype=torch.bfloat16, generator=g) for _ in range(3))
    o = torch.empty_like(q)
    lse = torch.empty(B, H, S, device="cuda", dtype=torch.float32)
    scale = 1.0 / math.sqrt(D)
    if family == "softmax":
        fn = lambda: hb.attn_fwd(q, k, v, family=hb.MA_ATTN_SOFTMAX, causal=causal, scale=scale, out=o, row_scale=lse)
    else:  # sigmoid(q.k*scale - log S)
        fn = lambda: hb.attn_fwd(q, k, v, family=hb.MA_ATTN_SIGMOID, causal=causal, scale=scale, bias=-math.log(S), out=o)
    ms = time_gpu(fn, steps, warmup)
    flops = (0.5 if causal else 1.0) * 4.0 * B * H * S * S * D
    return dict(ms=ms, flops=flops, tflops=flops / ms / 1e9, shape=dict(B=B, H=H, S=S, D=D, DV=D, causal=causal))


def bench_softmax_operator(steps, warmup):
    """The headline workload through the operator that AttentionEngine returns for the softmax spec (what a user of the
    reference calls: it allocates its output and lse, reads the current stream, goes through ctypes)."""
    import torch
    from attn_engine import AttentionEngine, OnlineFunc
    from core import CustomIO, SymbolicArray, SymbolScalar, Var, meta_tensor
    B, H, S, D = 8, 32, 4096, 128

    class OnlineSoftmax(OnlineFunc):   # the row function of examples/mha.py:21-71
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
            o_new = o / online_rowscales["r"]
            lse = online_rowscales["r"].log() + online_rowscales["m"]
            return o_new, {"lse": lse}

    meta = tuple(meta_tensor(B, H, S, D, dtype=torch.bfloat16) for _ in range(3))
    mod = AttentionEngine(meta, CustomIO({}), score_mod=lambda s, io, b, h, q, k: s * (D ** -0.5),
                          mask_mod=lambda b, h, q, k: q >= k, online_func=OnlineSoftmax())
    g = torch.Generator(device="cuda").manual_seed(0)
    q, k, v = (torch.randn(B, S, H, D, device="cuda", dtype=torch.bfloat16, generator=g) for _ in range(3))
    with torch.no_grad():
        ms = time_gpu(lambda: mod(q, k, v), steps, warmup)
    return _mfma_entry(ms, 0.5 * 4.0 * B * H * S * S * D, "the headline workload through the AttentionEngine operator (allocates o and lse per call)")


def bench_linear_operators(steps, warmup, which):
    """The chunked RetNet / Mamba2 workloads through the operator LinearAttentionEngine returns (reference call sites:
    testing/test.py:198-200 mod(C, B, x, dt, A, dt_bf16) and :776 mod(q, k, v, decay)): with the eager decay_mod / v_mod
    tensor work around the kernel, the output allocation and the workspace the operator keeps."""
    import torch
    from attn_engine import LinearAttentionEngine
    from core import CustomIO, meta_tensor
    g = torch.Generator(device="cuda").manual_seed(0)
    if which == "retnet":
        B, H, T, Dk, Dv = 8, 16, 2048, 256, 512
        meta = (meta_tensor(B, H, T, Dk, dtype=torch.bfloat16), meta_tensor(B, H, T, Dk, dtype=torch.bfloat16), meta_tensor(B, H, T, Dv, dtype=torch.bfloat16))
        mod = LinearAttentionEngine(meta, q_mod=lambda q, io: q * (Dk ** -0.5), decay_mod=lambda decay, io: decay.log(), custom_io=CustomIO({}))
        q = (torch.randn(B, H, T, Dk, device="cuda", generator=g) / 16).bfloat16()
        k = (torch.randn(B, H, T, Dk, device="cuda", generator=g) / 16).bfloat16()
        v = torch.randn(B, H, T, Dv, device="cuda", generator=g).bfloat16()
        decay = (1 - torch.exp2(-5 - torch.arange(H, device="cuda").float())).view(1, H, 1).expand(B, H, T).contiguous()
        with torch.no_grad():
            ms = time_gpu(lambda: mod(q, k, v, decay), steps, warmup)
        flops = B * H * (2.0 * T * 64 * (Dk + Dv) + 4.0 * T * Dk * Dv)
        return _mfma_entry(ms, flops, "c3_retnet_chunked through the LinearAttentionEngine operator (eager log of the decay, output allocation)")
    B, H, T, P, N = 8, 64, 2048, 64, 128
    meta = (meta_tensor(B, 1, T, N, dtype=torch.bfloat16), meta_tensor(B, 1, T, N, dtype=torch.bfloat16), meta_tensor(B, H, T, P, dtype=torch.bfloat16))
    io = CustomIO({"A": (1, "heads"), "dt": ("batch", "heads", "seq_len")})
    mod = LinearAttentionEngine(meta, decay_mod=lambda decay, io: decay * io.input_tensors["A"], v_mod=lambda v, io: v * io.input_tensors["dt"], custom_io=io)
    Cm = (torch.randn(B, 1, T, N, device="cuda", generator=g) / math.sqrt(N)).bfloat16()
    Bm = (torch.randn(B, 1, T, N, device="cuda", generator=g) / math.sqrt(N)).bfloat16()
    x = torch.randn(B, H, T, P, device="cuda", generator=g).bfloat16()
    dt = torch.nn.functional.softplus(torch.randn(B, H, T, device="cuda", generator=g) - 2)
    A = -torch.exp(torch.rand(1, H, device="cuda", generator=g) * math.log(16))
    dt16 = dt.bfloat16()
    with torch.no_grad():
        ms = time_gpu(lambda: mod(Cm, Bm, x, dt, A, dt16), steps, warmup)
    flops = B * H * (2.0 * T * 256 * N + 2.0 * T * 256 * P + 4.0 * T * N * P)
    return _mfma_entry(ms, flops, "c4_mamba2_ssd through the LinearAttentionEngine operator (eager dt * A, output allocation)")


def bench_retention_operator(steps, warmup):
    """c3_retnet_parallel through the operator AttentionEngine returns for the spec of examples/retention_parallel.py:25-111,
    called as testing/benchmark_h100.py:794-801 does: mod(q, k, v, mask) with the [1,H,S,S] bf16 decay mask.  The operator
    checks once per mask tensor (on the device) whether it is gamma_h^(i-j) below the diagonal, and then lets the kernel
    generate it."""
    import torch
    from attn_engine import AttentionEngine, OnlineFunc
    from core import CustomIO, SymbolScalar, Var, meta_tensor
    B, H, S, D, DV = 8, 16, 2048, 256, 512

    class OnlineRetention(OnlineFunc):   # examples/retention_parallel.py:36-86
        def __init__(self):
            super().__init__({"r_wo_clamp": SymbolScalar("r_wo_clamp", Var("0.0")), "r": SymbolScalar("r", Var("0.0"))},
                             {"r": SymbolScalar("r", Var("0.0"))}, CustomIO())

        @staticmethod
        def online_fwd(scores, rs, b, h, q_idx):
            r_wo_clamp = rs["r_wo_clamp"] + scores.get_reduce("abssum")
            r_new = r_wo_clamp.max(1.0)
            return scores / r_new, {"r_wo_clamp": r_wo_clamp, "r": r_new}, rs["r"] / r_new

        @staticmethod
        def online_fwd_epilogue(o, rs, b, h, q_idx):
            return o, {"r": rs["r"]}

    meta = (meta_tensor(B, H, S, D, dtype=torch.bfloat16), meta_tensor(B, H, S, D, dtype=torch.bfloat16), meta_tensor(B, H, S, DV, dtype=torch.bfloat16))
    mod = AttentionEngine(meta, CustomIO({"mask": (1, "heads", "seq_len", "seq_len_kv")}),
                          score_mod=lambda s, io, b, h, qi, ki: s * io.input_tensors["mask"], mask_mod=lambda b, h, qi, ki: qi >= ki,
                          online_func=OnlineRetention(), mask_value="0")
    g = torch.Generator(device="cuda").manual_seed(0)
    q = (torch.randn(B, S, H, D, device="cuda", generator=g) / 16).bfloat16()
    k = (torch.randn(B, S, H, D, device="cuda", generator=g) / 16).bfloat16()
    v = torch.randn(B, S, H, DV, device="cuda", generator=g).bfloat16()
    idx = torch.arange(S, device="cuda", dtype=torch.float32)
    gam = 1 - torch.exp2(-5 - torch.arange(H, device="cuda").float())
    diff = (idx.view(S, 1) - idx.view(1, S))
    mask = (torch.exp2(diff.clamp(min=0).unsqueeze(0) * torch.log2(gam).view(H, 1, 1)) * (diff >= 0)).unsqueeze(0).bfloat16()
    with torch.no_grad():
        mod(q, k, v, mask)            # the first call analyses the mask (once per mask tensor); its temporaries go back to the driver
        torch.cuda.synchronize()
        torch.cuda.empty_cache()
        ms = time_gpu(lambda: mod(q, k, v, mask), steps, warmup)
    generated = bool(getattr(mod, "last_call_generated_mask", False))
    return _mfma_entry(ms, 0.5 * 2.0 * B * H * S * S * (D + DV),
                       "c3_retnet_parallel through the AttentionEngine operator, mod(q, k, v, mask) with the [1,H,S,S] bf16 decay mask; "
                       "the operator found the mask to be gamma_h^(i-j) and the kernel generates it" if generated else
                       "c3_retnet_parallel through the AttentionEngine operator, mod(q, k, v, mask): the mask tensor is read")


def bench_mla_operator(steps, warmup):
    """c5_mla_decode through the operator AttentionEngine(kv_shared=True) returns (reference call site testing/test.py:842-848):
    mod(q, q_pe, kv, k_pe), with its output and workspace handling; cold, clean caches as for the C-ABI figure."""
    import torch
    from attn_engine import AttentionEngine, OnlineFunc
    from core import CustomIO, SymbolScalar, Var, meta_tensor
    B, Hq, Skv, D, Dpe = 64, 128, 4096, 512, 64

    class Online(OnlineFunc):   # (the MLA path takes the template's own softmax: lower_decode_mla.py:25-38)
        def __init__(self):
            super().__init__({"m": SymbolScalar("m", Var("-inf")), "r": SymbolScalar("r", Var("0.0"))},
                             {"lse": SymbolScalar("lse", Var("0.0"))}, CustomIO())

        @staticmethod
        def online_fwd(scores, rs, b, h, q_idx):
            m_new = rs["m"].max(scores.get_reduce("max"))
            c = (rs["m"] - m_new).exp()
            p = (scores - m_new).exp()
            return p, {"m": m_new, "r": rs["r"] * c + p.get_reduce("sum")}, c

        @staticmethod
        def online_fwd_epilogue(o, rs, b, h, q_idx):
            return o / rs["r"], {"lse": rs["r"].log() + rs["m"]}

    meta = (meta_tensor(B, Hq, 1, D + Dpe, dtype=torch.bfloat16), meta_tensor(B, 1, Skv, D + Dpe, dtype=torch.bfloat16),
            meta_tensor(B, 1, Skv, D, dtype=torch.bfloat16))
    mod = AttentionEngine(meta, CustomIO({}), score_mod=lambda s, io, b, h, qi, ki: s * ((D + Dpe) ** -0.5), mask_mod=None,
                          online_func=Online(), kv_shared=True)
    g = torch.Generator(device="cuda").manual_seed(0)
    q = torch.randn(B, 1, Hq, D, device="cuda", dtype=torch.bfloat16, generator=g)
    q_pe = torch.randn(B, 1, Hq, Dpe, device="cuda", dtype=torch.bfloat16, generator=g)
    kv = torch.randn(B, Skv, 1, D, device="cuda", dtype=torch.bfloat16, generator=g)
    k_pe = torch.randn(B, Skv, 1, Dpe, device="cuda", dtype=torch.bfloat16, generator=g)
    junk = _junk()
    with torch.no_grad():
        fn = lambda: mod(q, q_pe, kv, k_pe)
        ms_warm = time_gpu(fn, steps, warmup)
        ms_dirty = time_gpu(fn, steps, warmup, flush=lambda: junk.fill_(1))
        ms = time_gpu(fn, steps, warmup, flush=lambda: junk.sum())
    nbytes = 2.0 * (kv.numel() + k_pe.numel() + q.numel() + q_pe.numel() + q.numel())
    return dict(**_hbm_entry(ms, ms_dirty, ms_warm, nbytes), note="c5_mla_decode through the AttentionEngine(kv_shared=True) operator; " + COLD_NOTE)


def bench_softmax_bwd(steps, warmup):
    """Backward of the headline workload (dq, dk, dv given o, lse, do).  FLOPs by the usual convention:
    5 tile products against the forward's 2, causal at one half."""
    import torch
    from metaattention_amd import hip_backend as hb
    B, H, S, D = 8, 32, 4096, 128
    g = torch.Generator(device="cuda").manual_seed(0)
    q, k, v, do = (torch.randn(B, S, H, D, device="cuda", dtype=torch.bfloat16, generator=g) for _ in range(4))
    lse = torch.empty(B, H, S, device="cuda", dtype=torch.float32)
    scale = 1.0 / math.sqrt(D)
    o = hb.attn_fwd(q, k, v, family=hb.MA_ATTN_SOFTMAX, causal=True, scale=scale, row_scale=lse)
    ms = time_gpu(lambda: hb.attn_bwd(q, k, v, o, do, lse, family=hb.MA_ATTN_SOFTMAX, causal=True, scale=scale), max(steps // 3, 3), 2)
    flops = 2.5 * 0.5 * 4.0 * B * H * S * S * D
    return _mfma_entry(ms, flops, "backward, 2.5 x the forward's algorithmic FLOPs (5 tile products; the dq kernel and the fused dk/dv kernel execute 7: each recomputes the scores)")


def bench_decode(steps, warmup, B=64, H=32, Hkv=8, Skv=4096, D=128):
    """Grouped-query decode, one query token per sequence (HBM bound): the query heads of a kv head are handed to the
    kernel as the rows of that head, the cache is cut into kv splits."""
    import torch
    from metaattention_amd import hip_backend as hb
    g = torch.Generator(device="cuda").manual_seed(0)
    grp = H // Hkv
    q = torch.randn(B, 1, H, D, device="cuda", dtype=torch.bfloat16, generator=g)
    k = torch.randn(B, Skv, Hkv, D, device="cuda", dtype=torch.bfloat16, generator=g)
    v = torch.randn(B, Skv, Hkv, D, device="cuda", dtype=torch.bfloat16, generator=g)
    o = torch.empty_like(q)
    qv, ov = q.view(B, Hkv, grp, D).transpose(1, 2), o.view(B, Hkv, grp, D).transpose(1, 2)
    ws = torch.empty(1 << 26, dtype=torch.uint8, device="cuda")
    junk = _junk()
    fn = lambda: hb.attn_fwd(qv, k, v, family=hb.MA_ATTN_SOFTMAX, causal=False, scale=1 / math.sqrt(D), out=ov, workspace=ws)
    ms_warm = time_gpu(fn, steps, warmup)
    ms_dirty = time_gpu(fn, steps, warmup, flush=lambda: junk.fill_(1))
    ms = time_gpu(fn, steps, warmup, flush=lambda: junk.sum())   # (last: a kernel trace's last `steps` dispatches are these)
    nbytes = 2.0 * (k.numel() + v.numel() + q.numel() + o.numel())
    return dict(**_hbm_entry(ms, ms_dirty, ms_warm, nbytes),
                shape=dict(B=B, H=H, Hkv=Hkv, Sq=1, Skv=Skv, D=D), note="split-KV kernel + combine kernel per call; " + COLD_NOTE)


def bench_retnet_chunked(steps, warmup, backward=False):
    import torch
    from metaattention_amd import hip_backend as hb
    B, H, T, Dk, Dv = 8, 16, 2048, 256, 512
    g = torch.Generator(device="cuda").manual_seed(0)
    q = (torch.randn(B, H, T, Dk, device="cuda", generator=g) / 16).bfloat16()
    k = (torch.randn(B, H, T, Dk, device="cuda", generator=g) / 16).bfloat16()
    v = torch.randn(B, H, T, Dv, device="cuda", generator=g).bfloat16()
    ld = torch.log(1 - torch.exp2(-5 - torch.arange(H, device="cuda").float())).view(1, H, 1).expand(B, H, T).contiguous()
    C = 64
    flops = B * H * (2.0 * T * C * (Dk + Dv) + 4.0 * T * Dk * Dv)
    if backward:
        do = torch.randn(B, H, T, Dv, device="cuda", generator=g).bfloat16()
        ws = torch.empty(_linear_bwd_workspace(hb, B, H, H, H, T, Dk, Dv), dtype=torch.uint8, device="cuda")
        ms = time_gpu(lambda: hb.linear_bwd(q, k, v, ld, do, q_scale=Dk ** -0.5, workspace=ws), max(steps // 3, 3), 2)
        return _mfma_entry(ms, 2.5 * flops, "backward (dq, dk, dv, dlog_decay), 2.5 x the forward's algorithmic FLOPs; five scans of the "
                                            "forward kernel on operands read in place (the two 512-wide contractions as two pieces side by side) + epilogue")
    o = torch.empty_like(v)
    ws = torch.empty(max(hb.linear_workspace_bytes(B, H, H, H, T, Dk, Dv), 16), dtype=torch.uint8, device="cuda")
    ms = time_gpu(lambda: hb.linear_fwd(q, k, v, ld, q_scale=Dk ** -0.5, out=o, workspace=ws), steps, warmup)
    return _mfma_entry(ms, flops, "chunked form, chunk 64: 2*S*C*(Dqk+Dv) + 4*S*Dqk*Dv per (batch, head)")


def bench_retnet_parallel(steps, warmup, backward=False, generated_mask=False):
    import torch
    from metaattention_amd import hip_backend as hb
    B, H, S, D, DV = 8, 16, 2048, 256, 512
    g = torch.Generator(device="cuda").manual_seed(0)
    q = (torch.randn(B, S, H, D, device="cuda", generator=g) / 16).bfloat16()
    k = (torch.randn(B, S, H, D, device="cuda", generator=g) / 16).bfloat16()
    v = torch.randn(B, S, H, DV, device="cuda", generator=g).bfloat16()
    idx = torch.arange(S, device="cuda", dtype=torch.float32)
    gam = 1 - torch.exp2(-5 - torch.arange(H, device="cuda").float())
    diff = (idx.view(S, 1) - idx.view(1, S))
    mask = (torch.exp2(diff.clamp(min=0).unsqueeze(0) * torch.log2(gam).view(H, 1, 1)) * (diff >= 0)).unsqueeze(0).bfloat16()
    o = torch.empty_like(v)
    r = torch.empty(B, H, S, device="cuda")
    flops = 0.5 * 2.0 * B * H * S * S * (D + DV)
    if backward:
        hb.attn_fwd(q, k, v, family=hb.MA_ATTN_RETENTION, causal=True, scale=1.0, score_mask=mask, out=o, row_scale=r)
        do = torch.randn(B, S, H, DV, device="cuda", generator=g).bfloat16()
        mask_t = mask.transpose(2, 3).contiguous()
        ms = time_gpu(lambda: hb.attn_bwd(q, k, v, o, do, r, family=hb.MA_ATTN_RETENTION, causal=True, scale=1.0, score_mask=mask,
                                          score_mask_t=mask_t), max(steps // 3, 3), 2)
        return _mfma_entry(ms, 2.5 * flops, "backward, 2.5 x the forward's algorithmic FLOPs (three kernels dq, dv, dk)")
    if generated_mask:
        gamma = gam.contiguous()
        ms = time_gpu(lambda: hb.attn_fwd(q, k, v, family=hb.MA_ATTN_RETENTION, causal=True, scale=1.0, decay_gamma=gamma, out=o,
                                          row_scale=r), steps, warmup)
        return _mfma_entry(ms, flops, "parallel form, causal counted at one half; the decay mask gamma_h^(i-j) is generated by the kernel "
                                      "from the per-head gamma (decay_gamma) instead of being read as a [1,H,S,S] tensor")
    ms = time_gpu(lambda: hb.attn_fwd(q, k, v, family=hb.MA_ATTN_RETENTION, causal=True, scale=1.0, score_mask=mask, out=o,
                                      row_scale=r), steps, warmup)
    return _mfma_entry(ms, flops, "parallel form, causal counted at one half; the decay mask is a [1,H,S,S] bf16 tensor argument, as the "
                                  "reference's operator takes it")


def _linear_bwd_workspace(hb, B, H, Hq, Hk, T, Dk, Dv):
    import ctypes
    p = hb.LinearBwdParams()
    p.dtype, p.batch, p.heads, p.heads_q, p.heads_k, p.seqlen, p.dim_k, p.dim_v = hb.MA_BF16, B, H, Hq, Hk, T, Dk, Dv
    return max(hb.load_library().ma_linear_bwd_workspace_bytes(ctypes.byref(p)), 16)


def bench_mamba2(steps, warmup, backward=False):
    import torch
    from metaattention_amd import hip_backend as hb
    B, H, T, P, N = 8, 64, 2048, 64, 128
    g = torch.Generator(device="cuda").manual_seed(0)
    Cm = (torch.randn(B, 1, T, N, device="cuda", generator=g) / math.sqrt(N)).bfloat16()
    Bm = (torch.randn(B, 1, T, N, device="cuda", generator=g) / math.sqrt(N)).bfloat16()
    x = torch.randn(B, H, T, P, device="cuda", generator=g).bfloat16()
    dt = torch.nn.functional.softplus(torch.randn(B, H, T, device="cuda", generator=g) - 2)
    A = -torch.exp(torch.rand(1, H, device="cuda", generator=g) * math.log(16))
    ld = (dt * A.view(1, H, 1)).contiguous()
    Lc = 256
    flops = B * H * (2.0 * T * Lc * N + 2.0 * T * Lc * P + 4.0 * T * N * P)
    if backward:
        do = torch.randn(B, H, T, P, device="cuda", generator=g).bfloat16()
        ws = torch.empty(_linear_bwd_workspace(hb, B, H, 1, 1, T, N, P), dtype=torch.uint8, device="cuda")
        ms = time_gpu(lambda: hb.linear_bwd(Cm, Bm, x, ld, do, v_scale=dt, workspace=ws), max(steps // 3, 3), 2)
        return _mfma_entry(ms, 2.5 * flops, "backward (dC, dB, dx, dlog_decay, ddt-scale), 2.5 x the forward's algorithmic FLOPs; three scans "
                                            "of the forward kernel on operands read in place + epilogue")
    o = torch.empty_like(x)
    ws = torch.empty(max(hb.linear_workspace_bytes(B, H, 1, 1, T, N, P), 16), dtype=torch.uint8, device="cuda")
    ms = time_gpu(lambda: hb.linear_fwd(Cm, Bm, x, ld, v_scale=dt, out=o, workspace=ws), steps, warmup)
    return _mfma_entry(ms, flops, "chunk 256, C.B^T counted per head: 2*S*L*N + 2*S*L*P + 4*S*N*P per (batch, head); "
                                  "the kernel itself uses 32-token chunks and executes fewer FLOPs")


def bench_mla(steps, warmup):
    import torch
    from metaattention_amd import hip_backend as hb
    B, Hq, Skv, D, Dpe = 64, 128, 4096, 512, 64
    g = torch.Generator(device="cuda").manual_seed(0)
    q = torch.randn(B, 1, Hq, D, device="cuda", dtype=torch.bfloat16, generator=g)
    q_pe = torch.randn(B, 1, Hq, Dpe, device="cuda", dtype=torch.bfloat16, generator=g)
    kv = torch.randn(B, Skv, 1, D, device="cuda", dtype=torch.bfloat16, generator=g)
    k_pe = torch.randn(B, Skv, 1, Dpe, device="cuda", dtype=torch.bfloat16, generator=g)
    o = torch.empty_like(q)
    ws = torch.empty(max(hb.mla_workspace_bytes(B, Hq, Skv), 16), dtype=torch.uint8, device="cuda")
    junk = _junk()
    fn = lambda: hb.mla_decode(q, q_pe, kv, k_pe, scale=1 / math.sqrt(D + Dpe), out=o, workspace=ws)
    ms_warm = time_gpu(fn, steps, warmup)
    ms_dirty = time_gpu(fn, steps, warmup, flush=lambda: junk.fill_(1))
    ms = time_gpu(fn, steps, warmup, flush=lambda: junk.sum())   # (last: a kernel trace's last `steps` dispatches are these)
    nbytes = 2.0 * (kv.numel() + k_pe.numel() + q.numel() + q_pe.numel() + o.numel())
    flops = 2.0 * B * Hq * Skv * (D + Dpe + D)
    return dict(**_hbm_entry(ms, ms_dirty, ms_warm, nbytes), tflops=round(flops / ms / 1e9, 1),
                note="split-KV kernel + combine kernel per call; " + COLD_NOTE)


def bench_reference_shapes(steps, warmup):
    """The shapes for which the reference's tuned_config files record kernel latencies of its own templates (TileLang
    autotuner, warmup 10 / rep 10: tl_template/linear/linear_tl.py:229-233, tl_template/attn/mla_decode_tl.py:324-328), timed
    here back to back as the tuner times them.  `reference_ms` is what those files hold (other hardware: context, not a
    baseline for `vs_baseline`); for the chunked operators it is the sum of the state kernel (h) and the output kernel (o),
    which the one kernel here replaces."""
    import torch
    from metaattention_amd import hip_backend as hb
    out = {}
    g = torch.Generator(device="cuda").manual_seed(0)
    # MLA decode, fp16 (tuned_config/{H100,MI250}/mla_decode.json)
    for (B, Skv), ref in (((8, 2048), {"H100": 0.0329, "MI250": 0.1986}), ((1, 2048), {"MI250": 0.1779}), ((1, 4096), {"MI250": 0.2507}),
                          ((1, 8192), {"MI250": 0.4293}), ((8, 4096), {"MI250": 0.4117}), ((8, 8192), {"MI250": 0.7550})):
        Hq, D, Dpe = 128, 512, 64
        q = torch.randn(B, 1, Hq, D, device="cuda", dtype=torch.float16, generator=g)
        q_pe = torch.randn(B, 1, Hq, Dpe, device="cuda", dtype=torch.float16, generator=g)
        kv = torch.randn(B, Skv, 1, D, device="cuda", dtype=torch.float16, generator=g)
        k_pe = torch.randn(B, Skv, 1, Dpe, device="cuda", dtype=torch.float16, generator=g)
        o = torch.empty_like(q)
        ws = torch.empty(max(hb.mla_workspace_bytes(B, Hq, Skv), 16), dtype=torch.uint8, device="cuda")
        ms = time_gpu(lambda: hb.mla_decode(q, q_pe, kv, k_pe, scale=1 / math.sqrt(D + Dpe), out=o, workspace=ws), steps, warmup)
        out[f"mla_decode_fp16_b{B}_hq128_kv{Skv}"] = dict(ms=round(ms, 4), reference_ms=ref)
    # RetNet chunked forward, bf16 (tuned_config/{H100,MI250}/retention_linear_{h,o}.json)
    for (B, T), ref in (((8, 2048), {"H100 chunk 128": 2.44, "H100 chunk 64": 3.07, "MI250 chunk 64": 13.8}), ((1, 2048), {"H100 chunk 128": 0.260}),
                        ((8, 4096), {"MI250 chunk 64": 27.4})):
        H, Dk, Dv = 32, 256, 512
        q = (torch.randn(B, H, T, Dk, device="cuda", generator=g) / 16).bfloat16()
        k = (torch.randn(B, H, T, Dk, device="cuda", generator=g) / 16).bfloat16()
        v = torch.randn(B, H, T, Dv, device="cuda", generator=g).bfloat16()
        ld = torch.log(1 - torch.exp2(-5 - torch.arange(H, device="cuda").float())).view(1, H, 1).expand(B, H, T).contiguous()
        o = torch.empty_like(v)
        ws = torch.empty(max(hb.linear_workspace_bytes(B, H, H, H, T, Dk, Dv), 16), dtype=torch.uint8, device="cuda")
        ms = time_gpu(lambda: hb.linear_fwd(q, k, v, ld, q_scale=Dk ** -0.5, out=o, workspace=ws), steps, warmup)
        out[f"retnet_chunked_b{B}_h32_s{T}_256_512"] = dict(ms=round(ms, 4), reference_ms=ref)
    # Mamba2 SSD forward, bf16, 80 heads sharing one B / C head (tuned_config/{H100,MI250}/mamba2_{h,o}.json)
    for T, ref in ((2048, {"H100 chunk 128": 0.600, "MI250 chunk 64": 2.87}), (8192, {"H100 chunk 128": 2.25, "MI250 chunk 64": 12.1})):
        B, H, P, N = 8, 80, 64, 128
        Cm = (torch.randn(B, 1, T, N, device="cuda", generator=g) / math.sqrt(N)).bfloat16()
        Bm = (torch.randn(B, 1, T, N, device="cuda", generator=g) / math.sqrt(N)).bfloat16()
        x = torch.randn(B, H, T, P, device="cuda", generator=g).bfloat16()
        dt = torch.nn.functional.softplus(torch.randn(B, H, T, device="cuda", generator=g) - 2)
        A = -torch.exp(torch.rand(1, H, device="cuda", generator=g) * math.log(16))
        ld = (dt * A.view(1, H, 1)).contiguous()
        o = torch.empty_like(x)
        ws = torch.empty(max(hb.linear_workspace_bytes(B, H, 1, 1, T, N, P), 16), dtype=torch.uint8, device="cuda")
        ms = time_gpu(lambda: hb.linear_fwd(Cm, Bm, x, ld, v_scale=dt, out=o, workspace=ws), steps, warmup)
        out[f"mamba2_ssd_b8_hv80_s{T}_n128_p64"] = dict(ms=round(ms, 4), reference_ms=ref)
    out["note"] = ("reference_ms: tuned_latency fields of the reference's tuned_config/<GPU>/*.json, the only measured values in its tree "
                   "(H100 and MI250; per kernel, h + o summed for the chunked operators); ms: one call here, back to back, same shapes and dtypes")
    return out


def bench_reference_benchmark_shapes(steps, warmup):
    """Figures of the reference's own benchmarks that the five headline configurations do not cover (testing/benchmark_mi250.py:40-55,
    testing/benchmark_h100.py:112,129): causal softmax at the DeepSeek-V2-Lite head sizes (16 heads, Dqk 192, Dv 128, fp16),
    ReLU attention at the ViT-S head size (6 heads, 64 / 64, fp16) and gated retention at 64 / 64 and 256 / 256, forward and
    backward through the C ABI; one query token at the DeepSeek-V2-Lite sizes, the block-sparse grouped-query decode and the
    parallel retention at 32 heads and S = 4096 (benchmark_h100.py:63-65, 95-99, 151-156), forward.  The reference writes its own timings to CSV files at run time and holds none in the tree."""
    import torch
    from metaattention_amd import hip_backend as hb
    out = {}
    g = torch.Generator(device="cuda").manual_seed(0)
    for name, fam, causal, B, H, S, D, DV in (("softmax_causal_deepseek_v2_lite_b8_h16_s4096_192_128_fp16", hb.MA_ATTN_SOFTMAX, True, 8, 16, 4096, 192, 128),
                                              ("softmax_causal_b8_h12_s4096_128_256_fp16", hb.MA_ATTN_SOFTMAX, True, 8, 12, 4096, 128, 256),   # (benchmark_h100.py:87)
                                              ("relu_vit_s_b64_h6_s1024_64_64_fp16", hb.MA_ATTN_RELU, False, 64, 6, 1024, 64, 64)):
        q, k = (torch.randn(B, S, H, D, device="cuda", dtype=torch.float16, generator=g) for _ in range(2))
        v, do = (torch.randn(B, S, H, DV, device="cuda", dtype=torch.float16, generator=g) for _ in range(2))
        if fam == hb.MA_ATTN_RELU:
            k, v = k * 0.5, v * 0.5
        lse = torch.empty(B, H, S, device="cuda") if fam == hb.MA_ATTN_SOFTMAX else None
        o = torch.empty(B, S, H, DV, device="cuda", dtype=torch.float16)
        scale = D ** -0.5
        ms_f = time_gpu(lambda: hb.attn_fwd(q, k, v, family=fam, causal=causal, scale=scale, out=o, row_scale=lse), steps, warmup)
        ms_b = time_gpu(lambda: hb.attn_bwd(q, k, v, o, do, lse, family=fam, causal=causal, scale=scale), max(steps // 3, 3), 2)
        flops = (0.5 if causal else 1.0) * 2.0 * B * H * S * S * (D + DV)
        out[name] = dict(fwd_ms=round(ms_f, 4), fwd_tflops=round(flops / ms_f / 1e9, 1), bwd_ms=round(ms_b, 4),
                         bwd_tflops_2p5x=round(2.5 * flops / ms_b / 1e9, 1))
    # gated retention at the two head sizes of testing/benchmark_h100.py:112,129 (16 heads 64 / 64: the key width runs in the
    # 128-wide kernel; 40 heads 256 / 256), per-token log decay, forward and backward
    for B, H, Dk, Dv in ((8, 16, 64, 64), (8, 40, 256, 256), (64, 16, 64, 64)):      # (the last: the batch of benchmark_h100.py:110-113)
        T = 4096
        q = (torch.randn(B, H, T, Dk, device="cuda", generator=g) / 4).bfloat16()
        k = (torch.randn(B, H, T, Dk, device="cuda", generator=g) / 4).bfloat16()
        v, do = (torch.randn(B, H, T, Dv, device="cuda", generator=g).bfloat16() for _ in range(2))
        ld = torch.nn.functional.logsigmoid(torch.randn(B, H, T, device="cuda", generator=g) + 3.0)
        o = torch.empty_like(v)
        ws = torch.empty(max(hb.linear_workspace_bytes(B, H, H, H, T, Dk, Dv), 16), dtype=torch.uint8, device="cuda")
        ms_f = time_gpu(lambda: hb.linear_fwd(q, k, v, ld, q_scale=Dk ** -0.5, out=o, workspace=ws), steps, warmup)
        wsb = torch.empty(_linear_bwd_workspace(hb, B, H, H, H, T, Dk, Dv), dtype=torch.uint8, device="cuda")
        ms_b = time_gpu(lambda: hb.linear_bwd(q, k, v, ld, do, q_scale=Dk ** -0.5, workspace=wsb), max(steps // 3, 3), 2)
        out[f"gated_retention_b{B}_h{H}_s4096_{Dk}_{Dv}_bf16"] = dict(fwd_ms=round(ms_f, 4), bwd_ms=round(ms_b, 4))
        del q, k, v, do, o, ws, wsb
    torch.cuda.empty_cache()
    # one query token against a cache at the DeepSeek-V2-Lite head sizes (benchmark_h100.py:63-65), fp16
    B, H, Skv, D, DV = 8, 16, 8192, 192, 128
    q = torch.randn(B, 1, H, D, device="cuda", dtype=torch.float16, generator=g)
    k = torch.randn(B, Skv, H, D, device="cuda", dtype=torch.float16, generator=g)
    v = torch.randn(B, Skv, H, DV, device="cuda", dtype=torch.float16, generator=g)
    o = torch.empty(B, 1, H, DV, device="cuda", dtype=torch.float16)
    ms = time_gpu(lambda: hb.attn_fwd(q, k, v, family=hb.MA_ATTN_SOFTMAX, causal=False, scale=D ** -0.5, out=o), steps, warmup)
    out["softmax_decode_deepseek_v2_lite_b8_h16_kv8192_192_128_fp16"] = dict(ms=round(ms, 4), gbytes_per_s=round((k.numel() + v.numel()) * 2 / ms / 1e6, 1))
    # block-sparse grouped-query decode (benchmark_h100.py:151-156: 32 query heads on 8 kv heads, half of the 32-key blocks kept), fp16
    B, H, G, Skv, D = 8, 32, 8, 8192, 128
    q = torch.randn(B, 1, H, D, device="cuda", dtype=torch.float16, generator=g)
    k, v = (torch.randn(B, Skv, G, D, device="cuda", dtype=torch.float16, generator=g) for _ in range(2))
    bm = (torch.rand(B, G, Skv // 32, device="cuda", generator=g) < 0.5).to(torch.uint8)
    lens = torch.full((B,), Skv, dtype=torch.int32, device="cuda")
    o = torch.empty(B, H // G, G, D, device="cuda", dtype=torch.float16).transpose(1, 2)
    qv = q.view(B, G, H // G, D).transpose(1, 2)          # the query heads of a kv head as the rows of that head, as the operator passes them
    ms = time_gpu(lambda: hb.attn_fwd(qv, k, v, family=hb.MA_ATTN_SOFTMAX, causal=False, scale=D ** -0.5, kv_seqlens=lens, kv_block_mask=bm,
                                      kv_block_size=32), steps, warmup)
    out["sparse_gqa_decode_b8_h32_g8_kv8192_128_128_fp16"] = dict(ms=round(ms, 4), kept_blocks=round(float(bm.float().mean()), 3))
    del q, k, v, o
    torch.cuda.empty_cache()
    # normalised parallel retention at RetNet-6.7B's 32 heads and S = 4096 (benchmark_h100.py:95-99), bf16: the decay mask as the
    # [1, H, S, S] tensor the reference's operator takes (1 GiB), and generated by the kernel
    B, H, S, D, DV = 8, 32, 4096, 256, 512
    q = (torch.randn(B, S, H, D, device="cuda", generator=g) / 16).bfloat16()
    k = (torch.randn(B, S, H, D, device="cuda", generator=g) / 16).bfloat16()
    v = torch.randn(B, S, H, DV, device="cuda", generator=g).bfloat16()
    o = torch.empty_like(v)
    gam = 1 - torch.exp2(-5 - torch.arange(H, device="cuda").float())
    idx = torch.arange(S, device="cuda", dtype=torch.float32)
    diff = idx.view(S, 1) - idx.view(1, S)
    mask = torch.empty(1, H, S, S, device="cuda", dtype=torch.bfloat16)
    for h in range(H):                                     # (head by head: bounds the fp32 temporaries)
        mask[0, h] = (torch.exp2(diff.clamp(min=0) * torch.log2(gam[h])) * (diff >= 0)).bfloat16()
    flops = 0.5 * 2.0 * B * H * S * S * (D + DV)
    ms_t = time_gpu(lambda: hb.attn_fwd(q, k, v, family=hb.MA_ATTN_RETENTION, causal=True, scale=1.0, score_mask=mask, out=o), max(steps // 2, 3), 2)
    ms_g = time_gpu(lambda: hb.attn_fwd(q, k, v, family=hb.MA_ATTN_RETENTION, causal=True, scale=1.0, decay_gamma=gam, out=o), max(steps // 2, 3), 2)
    out["retention_parallel_b8_h32_s4096_256_512_bf16"] = dict(ms_mask_tensor=round(ms_t, 4), ms_generated_mask=round(ms_g, 4),
                                                               tflops_generated_mask=round(flops / ms_g / 1e9, 1))
    return out


def bench_head_sizes(steps, warmup):
    """The parallel kernels at every head size of the tile table (the reference's own list, testing/test.py:54-63,
    benchmark_h100.py:87,129, benchmark_mi250.py:40-46) x row-function family, causal, B4 H16 S4096 bf16: forward and
    backward side by side, so that a size which falls behind its neighbours shows."""
    import torch
    from metaattention_amd import hip_backend as hb
    global RAMP_MS
    B, H, S = 4, 16, 4096
    fams = {"softmax": hb.MA_ATTN_SOFTMAX, "sigmoid": hb.MA_ATTN_SIGMOID, "relu": hb.MA_ATTN_RELU}
    g = torch.Generator(device="cuda").manual_seed(0)
    ramp, out = RAMP_MS, {}
    RAMP_MS = min(ramp, 20.0)
    try:
        for D, DV in ((64, 64), (128, 128), (128, 256), (192, 128), (256, 256), (256, 512)):
            q, k = (torch.randn(B, S, H, D, device="cuda", dtype=torch.bfloat16, generator=g) for _ in range(2))
            v, do = (0.5 * torch.randn(B, S, H, DV, device="cuda", dtype=torch.bfloat16, generator=g) for _ in range(2))
            o = torch.empty(B, S, H, DV, device="cuda", dtype=torch.bfloat16)
            flops = 0.5 * 2.0 * B * H * S * S * (D + DV)
            for name, fam in fams.items():
                lse = torch.empty(B, H, S, device="cuda") if name == "softmax" else None
                kw = dict(family=fam, causal=True, scale=D ** -0.5, bias=-3.0 if name == "sigmoid" else 0.0)
                ms_f = time_gpu(lambda: hb.attn_fwd(q, k, v, out=o, row_scale=lse, **kw), max(steps // 3, 3), 2)
                ms_b = time_gpu(lambda: hb.attn_bwd(q, k, v, o, do, lse, **kw), max(steps // 5, 3), 1)
                out[f"{D}/{DV} {name}"] = dict(fwd_ms=round(ms_f, 4), fwd_tflops=round(flops / ms_f / 1e9, 1),
                                               bwd_ms=round(ms_b, 4), bwd_tflops=round(2.5 * flops / ms_b / 1e9, 1))
    finally:
        RAMP_MS = ramp
    out["note"] = "causal, B4 H16 S4096 bf16; forward: algorithmic FLOPs (causal at one half); backward: 2.5 x the forward's"
    return out


def cpu_baseline_softmax():
    """Oracle (restated PyTorch reference, fp32) on the host cores over a bounded
    sample: the whole headline workload once (B=8, H=32, S=4096, D=128, causal), about ten seconds."""
    import torch
    import oracle
    B, H, S, D = 8, 32, 4096, 128
    q, k, v = oracle.inputs.softmax_inputs(B, H, S, D, D, dtype=torch.bfloat16, seed=0)
    oracle.softmax_attention(q[:1, :, :1], k[:1, :, :1], v[:1, :, :1], causal=True)  # warm-up
    t0 = time.perf_counter()
    oracle.softmax_attention(q, k, v, causal=True)
    dt = time.perf_counter() - t0
    flops = 0.5 * 4.0 * B * H * S * S * D
    return dict(value=round(flops / dt / 1e12, 4), unit="TFLOP/s", cores=torch.get_num_threads(), kind="port",
                sample=f"B={B} of 8, H={H}, S={S}, D={D}, causal, fp32 oracle (restated PyTorch reference), {dt:.1f} s, "
                       f"os.cpu_count()={os.cpu_count()}")


def _timed(fn):
    t0 = time.perf_counter()
    fn()
    return time.perf_counter() - t0


def cpu_baseline_retention_parallel():
    """bench_utils.py:1158-1163 restated (oracle.retention_parallel), fp32, the whole workload."""
    import torch
    import oracle
    B, H, S, D, DV = 8, 16, 2048, 256, 512
    q, k, v, _ = oracle.inputs.retnet_inputs(B, H, S, D, DV, seed=0, layout="bshd")
    mask = oracle.retention_decay_mask(H, S)
    dt = _timed(lambda: oracle.retention_parallel(q, k, v, mask))
    flops = 0.5 * 2.0 * B * H * S * S * (D + DV)
    return dict(value=round(flops / dt / 1e12, 4), unit="TFLOP/s", cores=torch.get_num_threads(), kind="port",
                sample=f"B=8 of 8, H={H}, S={S}, Dqk={D}, Dv={DV}, fp32 oracle, {dt:.1f} s")


def cpu_baseline_retnet_chunked():
    """testing/test.py:738-747 restated (oracle.retnet_quadratic: what the reference's test checks the chunked operator
    against), fp32, four batch entries of the 8; priced by the same chunk-64 FLOP convention as the GPU number."""
    import torch
    import oracle
    B, H, T, Dk, Dv = 4, 16, 2048, 256, 512
    q, k, v, _ = oracle.inputs.retnet_inputs(B, H, T, Dk, Dv, seed=0)
    dt = _timed(lambda: oracle.retnet_quadratic(q, k, v))
    flops = B * H * (2.0 * T * 64 * (Dk + Dv) + 4.0 * T * Dk * Dv)
    return dict(value=round(flops / dt / 1e12, 4), unit="TFLOP/s", cores=torch.get_num_threads(), kind="port",
                sample=f"B=4 of 8, H={H}, S={T}, Dqk={Dk}, Dv={Dv}, fp32 oracle (quadratic form), {dt:.1f} s; credited with the chunk-64 "
                       "algorithmic FLOPs of the GPU figure")


def cpu_baseline_mamba2():
    """testing/test.py:206-343 restated (oracle.ssd_chunk_scan_combined, chunk 256), fp32, four batch entries of the 8."""
    import torch
    import oracle
    B, H, T, P, N, Lc = 4, 64, 2048, 64, 128, 256
    Cm, Bm, x, dtt, A = oracle.inputs.mamba2_inputs(B, H, T, P, N, seed=0)
    xs, dts = x.transpose(1, 2).contiguous(), dtt.transpose(1, 2).contiguous()
    Bs, Cs = Bm.transpose(1, 2).contiguous(), Cm.transpose(1, 2).contiguous()
    dt = _timed(lambda: oracle.ssd_chunk_scan_combined(xs, dts, A.view(-1), Bs, Cs, chunk_size=Lc))
    flops = B * H * (2.0 * T * Lc * N + 2.0 * T * Lc * P + 4.0 * T * N * P)
    return dict(value=round(flops / dt / 1e12, 4), unit="TFLOP/s", cores=torch.get_num_threads(), kind="port",
                sample=f"B=4 of 8, H={H}, S={T}, P={P}, N={N}, chunk {Lc}, fp32 oracle, {dt:.1f} s")


def cpu_baseline_mla():
    """testing/test.py:807-839 restated (oracle.mla_decode), fp32, the whole workload."""
    import torch
    import oracle
    B, Hq, Skv, D, Dpe = 64, 128, 4096, 512, 64
    q, q_pe, kv, k_pe = oracle.inputs.mla_inputs(B, Hq, Skv, D, Dpe, seed=0)
    dt = _timed(lambda: oracle.mla_decode(q, q_pe, kv, k_pe))
    nbytes = 2.0 * (kv.numel() + k_pe.numel() + q.numel() + q_pe.numel() + q.numel())
    return dict(value=round(nbytes / dt / 1e9, 2), unit="GB/s", cores=torch.get_num_threads(), kind="port",
                sample=f"B=64 of 64, Hq={Hq}, KV={Skv}, d={D}+{Dpe}, fp32 oracle, {dt:.1f} s; algorithmic bytes of the bf16 tensors over the time")


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=30)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--ramp-ms", type=float, default=RAMP_MS,
                    help="milliseconds every workload keeps the device busy before its warm-up launches (clock ramp after idle)")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="run 5 plain device-to-device copies of 1 GiB and exit (reference point for rocprofv3 "
                         "FETCH_SIZE / WRITE_SIZE counters)")
    ap.add_argument("--only", default="", help="comma list limiting the other workloads (e.g. 'mla'); 'none' skips them")
    args = ap.parse_args()
    globals()["RAMP_MS"] = max(args.ramp_ms, 0.0)
    if args.gpus != 1:
        print("bench.py: this build runs on ONE GPU; --gpus N with N > 1 is not supported "
              "(every unit of work is independent per batch*head, so a multi-GPU run would only shard the batch).",
              file=sys.stderr)
        sys.exit(2)
    import torch
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible; the HIP path has no CPU fallback", file=sys.stderr)
        sys.exit(3)

    if args.calibrate_copy:
        src = torch.ones(2 ** 30, dtype=torch.uint8, device="cuda")
        dst = torch.empty_like(src)
        for _ in range(5):
            dst.copy_(src)
        torch.cuda.synchronize()
        print(json.dumps({"calibration": "5 device-to-device copies", "bytes_read_per_copy": 2 ** 30, "bytes_written_per_copy": 2 ** 30}))
        return

    main_res = bench_softmax(args.steps, args.warmup, "softmax")
    ramp = RAMP_MS
    globals()["RAMP_MS"] = 0.0
    ms_no_ramp = bench_softmax(args.steps, args.warmup, "softmax")["ms"]   # the same launches right after the warm-up steps, no clock ramp
    globals()["RAMP_MS"] = ramp
    others = {}
    want = [w for w in args.only.split(",") if w]
    table = [("c2_sigmoid_causal", "sigmoid", lambda: (lambda r: _mfma_entry(r["ms"], r["flops"]))(bench_softmax(args.steps, args.warmup, "sigmoid"))),
             # the same kernel where an item is longer: how much of the headline's distance to the ceiling is the shape
             ("softmax_noncausal_s4096", "noncausal", lambda: (lambda r: _mfma_entry(r["ms"], r["flops"], "non-causal, B8 H32 S4096 D128"))(
                 bench_softmax(max(args.steps // 2, 3), 2, "softmax", causal=False))),
             ("softmax_causal_s16384", "s16384", lambda: (lambda r: _mfma_entry(r["ms"], r["flops"], "causal, B2 H32 S16384 D128"))(
                 bench_softmax(max(args.steps // 3, 3), 2, "softmax", B=2, S=16384))),
             ("c2_softmax_causal_operator", "operator", lambda: bench_softmax_operator(args.steps, args.warmup)),
             ("c2_softmax_causal_bwd", "bwd", lambda: bench_softmax_bwd(args.steps, args.warmup)),
             ("c3_retnet_chunked", "retnet", lambda: bench_retnet_chunked(args.steps, args.warmup)),
             ("c3_retnet_chunked_bwd", "retnet_bwd", lambda: bench_retnet_chunked(args.steps, args.warmup, backward=True)),
             ("c3_retnet_parallel", "retention", lambda: bench_retnet_parallel(args.steps, args.warmup)),
             ("c3_retnet_parallel_operator", "retention_operator", lambda: bench_retention_operator(args.steps, args.warmup)),
             ("c3_retnet_parallel_generated_mask", "retention_gamma", lambda: bench_retnet_parallel(args.steps, args.warmup, generated_mask=True)),
             ("c3_retnet_parallel_bwd", "retention_bwd", lambda: bench_retnet_parallel(args.steps, args.warmup, backward=True)),
             ("c4_mamba2_ssd", "mamba", lambda: bench_mamba2(args.steps, args.warmup)),
             ("c4_mamba2_bwd", "mamba_bwd", lambda: bench_mamba2(args.steps, args.warmup, backward=True)),
             ("c3_retnet_chunked_operator", "retnet_operator", lambda: bench_linear_operators(args.steps, args.warmup, "retnet")),
             ("c4_mamba2_ssd_operator", "mamba_operator", lambda: bench_linear_operators(args.steps, args.warmup, "mamba")),
             ("c5_mla_decode", "mla", lambda: bench_mla(args.steps, args.warmup)),
             ("c5_mla_decode_operator", "mla_operator", lambda: bench_mla_operator(args.steps, args.warmup)),
             ("gqa_decode", "decode", lambda: bench_decode(args.steps, args.warmup)),
             ("reference_shapes", "reference_shapes", lambda: bench_reference_shapes(args.steps, args.warmup)),
             ("reference_benchmark_shapes", "reference_benchmark", lambda: bench_reference_benchmark_shapes(args.steps, args.warmup)),
             ("head_sizes", "head_sizes", lambda: bench_head_sizes(args.steps, args.warmup))]
    cpu_legs = {"c3_retnet_chunked": cpu_baseline_retnet_chunked, "c3_retnet_parallel": cpu_baseline_retention_parallel,
                "c4_mamba2_ssd": cpu_baseline_mamba2, "c5_mla_decode": cpu_baseline_mla}
    for name, key, fn in table:
        if want and (want == ["none"] or not any(key.startswith(w) or w in name for w in want)):
            continue
        try:
            others[name] = fn()
        except Exception as e:     # (a workload that fails is reported in its place; the headline line is still printed)
            others[name] = {"error": f"{type(e).__name__}: {e}"}
            print(f"bench.py: workload {name} failed: {e!r}", file=sys.stderr)
        torch.cuda.empty_cache()
        if name in cpu_legs and not args.no_cpu_baseline and "error" not in others[name]:
            others[name]["cpu_baseline"] = cpu_legs[name]()

    traffic, traffic_from = profiled_traffic(ATTN_FWD_PROFILE, ATTN_FWD_KERNEL)
    line = {
        "metric": "fwd TFLOP/s + % bf16 MFMA peak (prefill/chunked); decode HBM GB/s % peak",
        "value": round(main_res["tflops"], 2),
        "unit": "TFLOP/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "clock_ramp_ms": RAMP_MS,   # device kept busy with the workload for this long before the warm-up steps (see time_gpu)
        "ms_per_step": round(main_res["ms"], 4),
        "ms_per_step_no_ramp": round(ms_no_ramp, 4),   # timed right after the warm-up launches, without the clock ramp (comparable with figures taken before the ramp existed)
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16", "data": "synthetic",
        "config": {"workload": "causal softmax MHA forward, bf16 in / fp32 accumulate, B=8 H=32 S=4096 D=128",
                   **main_res["shape"]},
        "roofline": {"bound": "mfma", "achieved": round(main_res["tflops"], 2), "peak": PEAK_BF16_TFLOPS,
                     "unit": "TFLOP/s", "frac": round(main_res["tflops"] / PEAK_BF16_TFLOPS, 4), "traffic": traffic,
                     "traffic_from": traffic_from, "kernel": ATTN_FWD_KERNEL, "flops_per_launch": main_res["flops"]},
        "cpu_baseline": None,
        "other_workloads": others,
    }
    if not args.no_cpu_baseline:
        line["cpu_baseline"] = cpu_baseline_softmax()
    print(json.dumps(line))


if __name__ == "__main__":
    main()
