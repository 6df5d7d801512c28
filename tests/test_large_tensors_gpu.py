"""Tensors beyond 4 GiB (and 2^31 elements) through every C-ABI entry point: batch entries on both sides of the 2 GiB and
4 GiB marks and at the far end must come out as when they are run alone (the same kernels on a one-entry copy, which the
other test files hold against the oracle), and one (batch, head) slice at the far end is held against the oracle directly.
The kernels address a (batch, head) plane with 32-bit offsets from a 64-bit base; this is the test of the 64-bit part."""
import math

import pytest
import torch

import oracle

pytestmark = pytest.mark.gpu


def _hb():
    from metaattention_amd import hip_backend as hb
    hb.load_library()
    return hb


def _need(gib):
    free, _ = torch.cuda.mem_get_info()
    if free < gib * 2 ** 30:
        pytest.skip(f"needs {gib} GiB of free device memory")


def _rnd(*shape, seed, gain=1.0, dtype=torch.bfloat16):
    g = torch.Generator(device="cuda").manual_seed(seed)
    out = torch.empty(*shape, device="cuda", dtype=dtype)
    for b in range(shape[0]):      # (entry by entry: bounds the fp32 temporary)
        out[b] = (torch.randn(*shape[1:], device="cuda", generator=g) * gain).to(dtype)
    return out


def _gib(t):
    return t.numel() * t.element_size() / 2 ** 30


@pytest.mark.parametrize("D,DV,B,H,family,causal", [(128, 128, 264, 32, "softmax", True), (64, 64, 272, 64, "relu", False),
                                                     (192, 128, 180, 32, "softmax", True)])
def test_parallel_attention_beyond_4_gib(D, DV, B, H, family, causal):
    hb = _hb()
    _need(60)
    S = 2048
    q, k = _rnd(B, S, H, D, seed=1), _rnd(B, S, H, D, seed=2, gain=0.5)
    v, do = _rnd(B, S, H, DV, seed=3, gain=0.5), _rnd(B, S, H, DV, seed=4, gain=0.5)
    assert _gib(q) > 4.0
    print(f"large {family} D{D}/{DV} B{B} H{H} S{S}: q {_gib(q):.2f} GiB", flush=True)
    fam = {"softmax": hb.MA_ATTN_SOFTMAX, "relu": hb.MA_ATTN_RELU}[family]
    lse = torch.empty(B, H, S, device="cuda") if family == "softmax" else None
    kw = dict(family=fam, causal=causal, scale=D ** -0.5)
    o = hb.attn_fwd(q, k, v, row_scale=lse, **kw)
    grads = hb.attn_bwd(q, k, v, o, do, lse, **kw)
    torch.cuda.synchronize()
    for b in (0, B // 2 - 1, B // 2, B - 1):
        one = lambda t: t[b:b + 1].contiguous()
        lse1 = torch.empty(1, H, S, device="cuda") if lse is not None else None
        o1 = hb.attn_fwd(one(q), one(k), one(v), row_scale=lse1, **kw)
        g1 = hb.attn_bwd(one(q), one(k), one(v), o1, one(do), lse1, **kw)
        torch.cuda.synchronize()
        assert torch.equal(o[b:b + 1], o1) and (lse is None or torch.equal(lse[b:b + 1], lse1)), f"entry {b}"
        for name, a, c in zip(("dq", "dk", "dv"), grads, g1):
            assert torch.equal(a[b:b + 1], c), f"entry {b}: {name}"
    cut = lambda t: t[B - 1:, :, H - 1:].cpu()
    ref = oracle.softmax_attention(cut(q), cut(k), cut(v), causal=causal) if family == "softmax" else oracle.relu_attention(cut(q), cut(k), cut(v))
    oracle.assert_close(cut(o).float(), ref, rtol=1e-2, atol=2e-2, mismatch_ratio=2e-2 if family == "relu" else 0.0)


@pytest.mark.parametrize("B,Hq,H,T,Dk,Dv", [(72, 16, 16, 4096, 256, 512), (80, 1, 64, 8192, 128, 64)])
def test_chunked_linear_attention_beyond_4_gib(B, Hq, H, T, Dk, Dv):
    """RetNet's and Mamba2's head layouts, forward and backward (the library may cut a lone entry into sequence segments
    and the batch not, so the comparison is to rounding, not to the bit)."""
    hb = _hb()
    _need(80)
    q, k = _rnd(B, Hq, T, Dk, seed=5, gain=1 / 16), _rnd(B, Hq, T, Dk, seed=6, gain=1 / 16)
    v, do = _rnd(B, H, T, Dv, seed=7), _rnd(B, H, T, Dv, seed=8, gain=0.5)
    ld = torch.nn.functional.logsigmoid(torch.randn(B, H, T, device="cuda", generator=torch.Generator(device="cuda").manual_seed(9)) + 3.0)
    assert _gib(v) > 4.0
    print(f"large linear B{B} H{H}/{Hq} T{T} Dk{Dk} Dv{Dv}: v {_gib(v):.2f} GiB", flush=True)
    o = hb.linear_fwd(q, k, v, ld, q_scale=Dk ** -0.5)
    grads = hb.linear_bwd(q, k, v, ld, do, q_scale=Dk ** -0.5)
    torch.cuda.synchronize()
    for b in (0, B // 2 - 1, B // 2, B - 1):
        one = lambda t: t[b:b + 1].contiguous()
        o1 = hb.linear_fwd(one(q), one(k), one(v), one(ld), q_scale=Dk ** -0.5)
        g1 = hb.linear_bwd(one(q), one(k), one(v), one(ld), one(do), q_scale=Dk ** -0.5)
        torch.cuda.synchronize()
        torch.testing.assert_close(o[b:b + 1].float(), o1.float(), rtol=1e-2, atol=1e-2, msg=f"entry {b}: o")
        for name, a, c in zip(("dq", "dk", "dv", "dlog_decay"), grads, g1):
            torch.testing.assert_close(a[b:b + 1].float(), c.float(), rtol=2e-2, atol=2e-2, msg=f"entry {b}: {name}")


def test_mla_decode_beyond_4_gib():
    hb = _hb()
    _need(20)
    B, Hq, Skv = 72, 16, 65536
    q, qp = _rnd(B, 1, Hq, 512, seed=10), _rnd(B, 1, Hq, 64, seed=11)
    kv, kp = _rnd(B, Skv, 1, 512, seed=12), _rnd(B, Skv, 1, 64, seed=13)
    assert _gib(kv) > 4.0
    print(f"large mla B{B} Hq{Hq} Skv{Skv}: kv {_gib(kv):.2f} GiB", flush=True)
    lse = torch.empty(B, Hq, device="cuda")
    o = hb.mla_decode(q, qp, kv, kp, scale=1 / math.sqrt(576), lse=lse)
    torch.cuda.synchronize()
    for b in (0, B // 2 - 1, B // 2, B - 1):
        one = lambda t: t[b:b + 1].contiguous()
        lse1 = torch.empty(1, Hq, device="cuda")
        o1 = hb.mla_decode(one(q), one(qp), one(kv), one(kp), scale=1 / math.sqrt(576), lse=lse1)
        torch.cuda.synchronize()
        torch.testing.assert_close(o[b:b + 1].float(), o1.float(), rtol=1e-2, atol=5e-3, msg=f"entry {b}")      # (other split counts)
        torch.testing.assert_close(lse[b:b + 1], lse1, rtol=1e-4, atol=1e-4)
    ref, lse_ref = oracle.mla_decode(q[B - 1:].cpu(), qp[B - 1:].cpu(), kv[B - 1:].cpu(), kp[B - 1:].cpu(), return_lse=True)
    oracle.assert_close(o[B - 1:].float().cpu(), ref, rtol=1e-2, atol=2e-2)
    torch.testing.assert_close(lse[B - 1:].cpu(), lse_ref, rtol=1e-4, atol=1e-4)
