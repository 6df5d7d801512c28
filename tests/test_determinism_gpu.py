"""Run-to-run determinism: no kernel of the library accumulates through atomics (dq has a kernel of its own, the kv splits
and the head groups are merged by reduction kernels in a fixed order), so the same call gives the same bits every time,
whatever ran in between."""
import math

import pytest
import torch

pytestmark = pytest.mark.gpu


def _hb():
    from metaattention_amd import hip_backend as hb
    hb.load_library()
    return hb


def _same(a, b):
    return all((x is None and y is None) or torch.equal(x, y) for x, y in zip(a, b))


def test_every_operator_is_bit_reproducible():
    hb = _hb()
    g = torch.Generator(device="cuda").manual_seed(3)
    rnd = lambda *s, dt=torch.bfloat16, gain=1.0: (gain * torch.randn(*s, device="cuda", generator=g)).to(dt)
    jobs = {}

    for D, DV, dt in ((128, 128, torch.bfloat16), (64, 64, torch.float16), (192, 128, torch.float16), (128, 256, torch.bfloat16), (256, 256, torch.bfloat16)):
        q, k, v, do = rnd(2, 777, 6, D, dt=dt), rnd(2, 777, 3, D, dt=dt, gain=0.5), rnd(2, 777, 3, DV, dt=dt, gain=0.5), rnd(2, 777, 6, DV, dt=dt)

        def parallel(q=q, k=k, v=v, do=do, D=D):
            lse = torch.empty(2, 6, 777, device="cuda")
            o = hb.attn_fwd(q, k, v, family=hb.MA_ATTN_SOFTMAX, causal=True, scale=D ** -0.5, row_scale=lse)
            return (o, lse) + tuple(hb.attn_bwd(q, k, v, o, do, lse, family=hb.MA_ATTN_SOFTMAX, causal=True, scale=D ** -0.5))
        jobs[f"softmax {D}/{DV}"] = parallel

    q, k, v = rnd(4, 1, 32, 128), rnd(4, 5000, 8, 128), rnd(4, 5000, 8, 128)
    lens = torch.tensor([5000, 17, 2048, 4999], dtype=torch.int32, device="cuda")
    jobs["decode with kv splits"] = lambda: (hb.attn_fwd(q.view(4, 8, 4, 128).transpose(1, 2), k, v, family=hb.MA_ATTN_SOFTMAX, causal=False,
                                                         scale=128 ** -0.5, kv_seqlens=lens),)

    ql, kl, vl, dol = rnd(2, 1, 1000, 128, gain=0.1), rnd(2, 1, 1000, 128, gain=0.1), rnd(2, 16, 1000, 64), rnd(2, 16, 1000, 64)
    ld = torch.nn.functional.logsigmoid(torch.randn(2, 16, 1000, device="cuda", generator=g) + 3.0)
    vs = torch.rand(2, 16, 1000, device="cuda", generator=g) + 0.5
    jobs["linear, shared q / k heads"] = lambda: (hb.linear_fwd(ql, kl, vl, ld, q_scale=1.0, v_scale=vs),) + tuple(hb.linear_bwd(ql, kl, vl, ld, dol, q_scale=1.0, v_scale=vs))
    qr, kr, vr, dor = rnd(1, 3, 700, 256, gain=1 / 16), rnd(1, 3, 700, 256, gain=1 / 16), rnd(1, 3, 700, 512), rnd(1, 3, 700, 512)
    ldr = torch.nn.functional.logsigmoid(torch.randn(1, 3, 700, device="cuda", generator=g) + 3.0)
    jobs["linear 256/512"] = lambda: (hb.linear_fwd(qr, kr, vr, ldr, q_scale=1 / 16),) + tuple(hb.linear_bwd(qr, kr, vr, ldr, dor, q_scale=1 / 16))

    qm, qpm, kvm, kpm = rnd(6, 1, 128, 512), rnd(6, 1, 128, 64), rnd(6, 4096, 1, 512), rnd(6, 4096, 1, 64)

    def mla():
        lse = torch.empty(6, 128, device="cuda")
        return (hb.mla_decode(qm, qpm, kvm, kpm, scale=1 / math.sqrt(576), lse=lse), lse)
    jobs["mla"] = mla

    first = {name: job() for name, job in jobs.items()}
    torch.cuda.synchronize()
    for rounds in range(3):
        for name in reversed(list(jobs)):       # another order: other neighbours in time and other recycled buffers
            got = jobs[name]()
            torch.cuda.synchronize()
            assert _same(got, first[name]), f"{name}: run {rounds + 2} differs from the first"
