"""The library keeps no state between calls (what it caches per kernel, the LDS opt-in and the occupancy, is written once
and atomically), and the binding launches on the calling thread's current stream: calls from several host threads, each on
a stream of its own, give the same bits as the same calls one after the other."""
import math
import threading

import pytest
import torch

pytestmark = pytest.mark.gpu


def _hb():
    from metaattention_amd import hip_backend as hb
    hb.load_library()
    return hb


def test_calls_from_four_threads_on_four_streams():
    hb = _hb()
    g = torch.Generator(device="cuda").manual_seed(0)
    rnd = lambda *s, dt=torch.bfloat16, gain=1.0: (gain * torch.randn(*s, device="cuda", generator=g)).to(dt)

    q1, k1, v1, do1 = rnd(2, 1024, 8, 128), rnd(2, 1024, 8, 128), rnd(2, 1024, 8, 128), rnd(2, 1024, 8, 128)

    def softmax_fwd_bwd():
        lse = torch.empty(2, 8, 1024, device="cuda")
        o = hb.attn_fwd(q1, k1, v1, family=hb.MA_ATTN_SOFTMAX, causal=True, scale=128 ** -0.5, row_scale=lse)
        return (o, lse) + tuple(hb.attn_bwd(q1, k1, v1, o, do1, lse, family=hb.MA_ATTN_SOFTMAX, causal=True, scale=128 ** -0.5))

    q2, k2, v2 = rnd(3, 700, 6, 64, dt=torch.float16), rnd(3, 900, 3, 64, dt=torch.float16, gain=0.5), rnd(3, 900, 3, 64, dt=torch.float16, gain=0.5)

    def relu_wide():
        return (hb.attn_fwd(q2, k2, v2, family=hb.MA_ATTN_RELU, causal=False, scale=0.125),)

    q3, k3, v3 = rnd(2, 1, 1024, 128, gain=0.1), rnd(2, 1, 1024, 128, gain=0.1), rnd(2, 16, 1024, 64)
    ld3 = torch.nn.functional.logsigmoid(torch.randn(2, 16, 1024, device="cuda", generator=g) + 3.0)
    vs3 = torch.rand(2, 16, 1024, device="cuda", generator=g) + 0.5

    def mamba_like():
        o = hb.linear_fwd(q3, k3, v3, ld3, q_scale=1.0, v_scale=vs3)
        return (o,) + tuple(t for t in hb.linear_bwd(q3, k3, v3, ld3, v3, q_scale=1.0, v_scale=vs3))

    q4, qp4, kv4, kp4 = rnd(8, 1, 128, 512), rnd(8, 1, 128, 64), rnd(8, 3000, 1, 512), rnd(8, 3000, 1, 64)

    def mla():
        lse = torch.empty(8, 128, device="cuda")
        return (hb.mla_decode(q4, qp4, kv4, kp4, scale=1 / math.sqrt(576), lse=lse), lse)

    jobs = [softmax_fwd_bwd, relu_wide, mamba_like, mla]
    serial = [job() for job in jobs]
    torch.cuda.synchronize()
    errors = []

    def worker(i):
        try:
            stream = torch.cuda.Stream()
            with torch.cuda.stream(stream):
                for it in range(12):
                    got = jobs[i]()
                    stream.synchronize()
                    for a, b in zip(got, serial[i]):
                        if not torch.equal(a, b):
                            errors.append(f"job {i} iteration {it}: result differs from the serial call")
                            return
        except Exception as e:      # (reported by the main thread)
            errors.append(f"job {i}: {e!r}")

    threads = [threading.Thread(target=worker, args=(i,)) for i in range(len(jobs))]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    torch.cuda.synchronize()
    assert not errors, errors
