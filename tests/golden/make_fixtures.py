"""Writes the golden vectors kept in this directory (``python tests/golden/make_fixtures.py``).

The reference ships no stored vectors for these operators (its tests compare
against PyTorch at run time), so the vectors here are computed from the
operators' *definitions* in fp64 numpy, element by element or token by token,
by code that shares nothing with ``oracle/`` (no tiling, no chunking, no torch
kernels).  ``tests/test_golden.py`` checks the oracle against them on the CPU
and the HIP operators against them on the GPU.

Inputs are seeded numpy normals rounded once to bf16 and stored as the bf16
bit patterns (uint16); expected outputs are fp32.  Definitions follow
  softmax   testing/test.py:79-104        sigmoid  testing/test.py:519-543
  relu      testing/test.py:599-604       retention (normalised) bench_utils.py:1158-1163
  RetNet    testing/test.py:738-747       gated retention testing/test.py:436-481
  Mamba2    testing/test.py:206-343 (as the state-space recurrence it discretises)
  MLA       testing/test.py:807-839
"""
import math
import os

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))


def bf16_round(x):
    """fp32 -> nearest-even bf16, returned as (uint16 bit patterns, float64 values)."""
    x = np.asarray(x, dtype=np.float32)
    u = x.view(np.uint32).astype(np.uint64)
    u = (u + 0x7FFF + ((u >> 16) & 1)) >> 16
    bits = u.astype(np.uint16)
    val = (bits.astype(np.uint32) << 16).view(np.float32).astype(np.float64)
    return bits, val


def normal(rng, *shape, gain=1.0):
    return bf16_round(rng.standard_normal(shape).astype(np.float32) * gain)


def softmax_case(rng, B, H, S, D, causal, DV=None):
    DV = DV or D
    (qb, q), (kb, k), (vb, v) = normal(rng, B, S, H, D), normal(rng, B, S, H, D), normal(rng, B, S, H, DV)
    out = np.zeros((B, S, H, DV))
    lse = np.zeros((B, H, S))
    for b in range(B):
        for h in range(H):
            for i in range(S):
                n = i + 1 if causal else S
                s = (k[b, :n, h] @ q[b, i, h]) / math.sqrt(D)
                m = s.max()
                e = np.exp(s - m)
                lse[b, h, i] = m + math.log(e.sum())
                out[b, i, h] = (e / e.sum()) @ v[b, :n, h]
    return dict(q=qb, k=kb, v=vb, out=out.astype(np.float32), lse=lse.astype(np.float32), causal=np.int32(causal))


def sigmoid_case(rng, B, H, S, D, bias, scale):
    (qb, q), (kb, k), (vb, v) = normal(rng, B, S, H, D), normal(rng, B, S, H, D), normal(rng, B, S, H, D)
    out = np.zeros((B, S, H, D))
    for b in range(B):
        for h in range(H):
            for i in range(S):
                s = (k[b, :i + 1, h] @ q[b, i, h]) * scale + bias
                out[b, i, h] = (1.0 / (1.0 + np.exp(-s))) @ v[b, :i + 1, h]
    return dict(q=qb, k=kb, v=vb, out=out.astype(np.float32), bias=np.float32(bias), scale=np.float32(scale))


def relu_case(rng, B, H, S, D):
    # keys and values at 0.5 as in testing/test.py:609-610
    (qb, q), (kb, k), (vb, v) = normal(rng, B, S, H, D), normal(rng, B, S, H, D, gain=0.5), normal(rng, B, S, H, D, gain=0.5)
    out = np.zeros((B, S, H, D))
    for b in range(B):
        for h in range(H):
            for i in range(S):
                out[b, i, h] = np.maximum((k[b, :, h] @ q[b, i, h]) / math.sqrt(D), 0.0) @ v[b, :, h]
    return dict(q=qb, k=kb, v=vb, out=out.astype(np.float32))


def retention_case(rng, B, H, S, D, DV, q_gain):
    (qb, q), (kb, k) = normal(rng, B, S, H, D, gain=q_gain / math.sqrt(D)), normal(rng, B, S, H, D, gain=1 / math.sqrt(D))
    vb, v = normal(rng, B, S, H, DV)
    gam = 1.0 - 2.0 ** (-5.0 - np.arange(H))
    mask = np.zeros((1, H, S, S), dtype=np.float32)
    for h in range(H):
        for i in range(S):
            mask[0, h, i, :i + 1] = gam[h] ** (i - np.arange(i + 1))
    mb, m = bf16_round(mask)
    out = np.zeros((B, S, H, DV))
    r = np.zeros((B, H, S))
    for b in range(B):
        for h in range(H):
            for i in range(S):
                s = (k[b, :, h] @ q[b, i, h]) * m[0, h, i]
                r[b, h, i] = max(np.abs(s).sum(), 1.0)
                out[b, i, h] = (s / r[b, h, i]) @ v[b, :, h]
    return dict(q=qb, k=kb, v=vb, mask=mb, out=out.astype(np.float32), r=r.astype(np.float32))


def recurrent_case(rng, B, Hq, H, T, DK, DV, kind):
    """o_t = q_scale * q_t S_t,  S_t = exp(g_t) S_{t-1} + k_t^T (v_t * vs_t), one token at a time.
    kind 'retnet': g_t = log(gamma_h); 'gated': g_t = log-sigmoid of a normal; 'mamba2': g_t = dt_t A_h, vs_t = dt_t."""
    # un-normalised operators: keys at 0.1 as in testing/test.py:750-756 keep the outputs O(1)
    qg, kg = (1 / math.sqrt(DK), 1 / math.sqrt(DK)) if kind == "mamba2" else (1.0, 0.1)
    (qb, q), (kb, k) = normal(rng, B, Hq, T, DK, gain=qg), normal(rng, B, Hq, T, DK, gain=kg)
    vb, v = normal(rng, B, H, T, DV)
    vs = None
    if kind == "retnet":
        g = np.broadcast_to(np.log(1.0 - 2.0 ** (-5.0 - np.arange(H)))[None, :, None], (B, H, T)).astype(np.float32)
        q_scale = DK ** -0.5
    elif kind == "gated":
        z = rng.standard_normal((B, H, T)) + 3.0
        g = (-np.log1p(np.exp(-z))).astype(np.float32)
        q_scale = DK ** -0.5
    else:
        dt = np.log1p(np.exp(rng.standard_normal((B, H, T)) - 2.0)).astype(np.float32)
        A = (-np.exp(rng.random(H) * math.log(16.0))).astype(np.float32)
        g = (dt.astype(np.float64) * A[None, :, None]).astype(np.float32)
        vs, q_scale = dt, 1.0
    out = np.zeros((B, H, T, DV))
    rep = H // Hq
    for b in range(B):
        for h in range(H):
            S = np.zeros((DK, DV))
            for t in range(T):
                vt = v[b, h, t] * (float(vs[b, h, t]) if vs is not None else 1.0)
                S = math.exp(float(g[b, h, t])) * S + np.outer(k[b, h // rep, t], vt)
                out[b, h, t] = q_scale * (q[b, h // rep, t] @ S)
    d = dict(q=qb, k=kb, v=vb, log_decay=g, out=out.astype(np.float32), q_scale=np.float32(q_scale))
    if vs is not None:
        d["v_scale"], d["A"] = vs, A
    return d


def mla_case(rng, B, Hq, Skv, D, DPE):
    (qb, q), (pb, qp) = normal(rng, B, 1, Hq, D), normal(rng, B, 1, Hq, DPE)
    (cb, kv), (eb, kp) = normal(rng, B, Skv, 1, D), normal(rng, B, Skv, 1, DPE)
    out = np.zeros((B, 1, Hq, D))
    lse = np.zeros((B, Hq))
    for b in range(B):
        for h in range(Hq):
            s = (kv[b, :, 0] @ q[b, 0, h] + kp[b, :, 0] @ qp[b, 0, h]) / math.sqrt(D + DPE)
            m = s.max()
            e = np.exp(s - m)
            lse[b, h] = m + math.log(e.sum())
            out[b, 0, h] = (e / e.sum()) @ kv[b, :, 0]
    return dict(q=qb, q_pe=pb, kv=cb, k_pe=eb, out=out.astype(np.float32), lse=lse.astype(np.float32))


CASES = {
    "softmax_causal_b1h2s160d128": lambda r: softmax_case(r, 1, 2, 160, 128, True),
    "softmax_full_b1h1s96d64": lambda r: softmax_case(r, 1, 1, 96, 64, False),
    "sigmoid_causal_b1h2s160d128": lambda r: sigmoid_case(r, 1, 2, 160, 128, -math.log(160.0), 1 / math.sqrt(128)),
    "relu_b1h2s130d128": lambda r: relu_case(r, 1, 2, 130, 128),
    "retention_parallel_b1h2s136": lambda r: retention_case(r, 1, 2, 136, 256, 512, 4.0),
    "retnet_b1h2t160": lambda r: recurrent_case(r, 1, 2, 2, 160, 256, 512, "retnet"),
    "gated_retention_b1h2t128": lambda r: recurrent_case(r, 1, 2, 2, 128, 128, 128, "gated"),
    "mamba2_b1h4t256": lambda r: recurrent_case(r, 1, 1, 4, 256, 128, 64, "mamba2"),
    "mla_b2h20s200": lambda r: mla_case(r, 2, 20, 200, 512, 64),
    # DeepSeek-V2-Lite's head sizes (testing/benchmark_mi250.py:40-55) and a 64-wide gated retention (testing/benchmark_h100.py:112)
    "softmax_causal_b1h2s144d192dv128": lambda r: softmax_case(r, 1, 2, 144, 192, True, DV=128),
    "gated_retention_b1h2t128dk64": lambda r: recurrent_case(r, 1, 2, 2, 128, 64, 64, "gated"),
}


def main():
    for i, (name, fn) in enumerate(CASES.items()):
        data = fn(np.random.default_rng(1000 + i))
        path = os.path.join(HERE, name + ".npz")
        np.savez_compressed(path, **data)
        print(f"{name}: {os.path.getsize(path) / 1024:.0f} KiB")


if __name__ == "__main__":
    main()
