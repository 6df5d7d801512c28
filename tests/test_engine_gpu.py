"""The operators AttentionEngine returns for user specs, called with the
reference's layouts and argument order, against the CPU oracle."""
import math

import pytest
import torch

import oracle
from oracle import inputs
import specs

pytestmark = pytest.mark.gpu
ATOL, RTOL = 2e-2, 1e-2


@pytest.mark.parametrize("online", ["plain", "respelled"])
def test_softmax_operator(online):
    B, H, S, D = 1, 4, 512, 128
    mod = specs.softmax_attention(B, H, S, D, D, online=specs.OnlineSoftmaxRespelled() if online == "respelled" else None)
    q, k, v = inputs.softmax_inputs(B, H, S, D, D, seed=1)
    o = mod(q.cuda(), k.cuda(), v.cuda())
    torch.cuda.synchronize()
    assert o.shape == (B, S, H, D) and o.dtype == torch.bfloat16
    ref, lse = oracle.softmax_attention(q, k, v, causal=True, return_lse=True)
    oracle.assert_close(o.float().cpu(), ref, rtol=RTOL, atol=ATOL)
    torch.testing.assert_close(mod.final_rowscales.cpu(), lse, rtol=1e-4, atol=1e-4)


def test_softmax_operator_fp16_noncausal():
    B, H, S, D = 2, 2, 256, 128
    mod = specs.softmax_attention(B, H, S, D, D, dtype=torch.float16, causal=False)
    q, k, v = inputs.softmax_inputs(B, H, S, D, D, dtype=torch.float16, seed=2)
    o = mod(q.cuda(), k.cuda(), v.cuda())
    torch.cuda.synchronize()
    oracle.assert_close(o.float().cpu(), oracle.softmax_attention(q, k, v, causal=False), rtol=RTOL, atol=ATOL)


def test_softmax_that_scales_the_scores_itself():
    """examples/mha_v2.py:15-99: score_mod returns the raw score, the online function computes exp2((s - m) * scale * log2 e)
    and lse = log r + scale * m.  The same operator as the usual spelling: output, lse and gradients bit for bit, and the
    oracle's values."""
    B, H, S, D = 1, 4, 384, 128
    mod, usual = specs.softmax_attention_inner_scale(B, H, S, D, D), specs.softmax_attention(B, H, S, D, D)
    assert mod.score_form.scale == usual.score_form.scale
    q, k, v = inputs.softmax_inputs(B, H, S, D, D, seed=21)
    got, exp = [], []
    for m, out in ((mod, got), (usual, exp)):
        qq, kk, vv = (t.cuda().requires_grad_(True) for t in (q, k, v))
        o = m(qq, kk, vv)
        o.backward(torch.ones_like(o) * 0.25)
        torch.cuda.synchronize()
        out += [o.detach(), m.final_rowscales, qq.grad, kk.grad, vv.grad]
    for a, b in zip(got, exp):
        assert torch.equal(a, b)
    ref, lse = oracle.softmax_attention(q, k, v, causal=True, return_lse=True)
    oracle.assert_close(got[0].float().cpu(), ref, rtol=RTOL, atol=ATOL)
    torch.testing.assert_close(got[1].cpu(), lse, rtol=1e-4, atol=1e-4)


def test_no_online_function_is_the_identity_row_function():
    """examples/sigmoid_attn_v2.py:62-68, reluattn_v2.py:54-60 pass online_func=None."""
    B, H, S, D = 1, 2, 256, 128
    mod = specs.sigmoid_attention(B, H, S, D, D, online=None)
    assert mod.family == "sigmoid"
    q, k, v = inputs.softmax_inputs(B, H, S, D, D, seed=22)
    q = (q.float() * 0.3).bfloat16()
    bias = torch.tensor([-4.25])
    o = mod(q.cuda(), k.cuda(), v.cuda(), bias.cuda())
    torch.cuda.synchronize()
    oracle.assert_close(o.float().cpu(), oracle.sigmoid_attention(q, k, v, bias, causal=True), rtol=RTOL, atol=ATOL, mismatch_ratio=2e-3)


def test_sigmoid_operator_with_bias_tensor():
    """mod(q, k, v, softmax_bias[1]) as in testing/test.py:552-566."""
    B, H, S, D = 1, 2, 256, 128
    mod = specs.sigmoid_attention(B, H, S, D, D)
    q, k, v = inputs.softmax_inputs(B, H, S, D, D, seed=3)
    q = (q.float() * 0.3).bfloat16()
    bias = torch.tensor([-4.25])
    o = mod(q.cuda(), k.cuda(), v.cuda(), bias.cuda())
    torch.cuda.synchronize()
    oracle.assert_close(o.float().cpu(), oracle.sigmoid_attention(q, k, v, bias, causal=True), rtol=RTOL, atol=ATOL, mismatch_ratio=2e-3)


def test_sigmoid_operator_scaled_constant_bias():
    """The benchmark's variant: sigmoid(q.k * scale - log S), written with exp()."""
    B, H, S, D = 1, 2, 512, 128
    mod = specs.sigmoid_attention(B, H, S, D, D, scale=D ** -0.5, const_bias=-math.log(S), form="exp")
    q, k, v = inputs.softmax_inputs(B, H, S, D, D, seed=4)
    o = mod(q.cuda(), k.cuda(), v.cuda())
    torch.cuda.synchronize()
    ref = oracle.sigmoid_attention(q, k, v, -math.log(S), causal=True, softmax_scale=D ** -0.5)
    oracle.assert_close(o.float().cpu(), ref, rtol=RTOL, atol=ATOL)


def test_outputs_carry_a_grad_fn_and_backward_runs():
    """The operator is a torch.autograd.Function.apply (attn_tl.py:694): outputs carry grad_fn, backward fills
    q.grad / k.grad / v.grad (values are checked in test_attn_bwd_gpu.py)."""
    B, H, S, D = 1, 1, 128, 128
    mod = specs.softmax_attention(B, H, S, D, D)
    q, k, v = (t.cuda().requires_grad_(True) for t in inputs.softmax_inputs(B, H, S, D, D, seed=5))
    o = mod(q, k, v)
    assert o.grad_fn is not None
    o.float().sum().backward()
    torch.cuda.synchronize()
    for t in (q, k, v):
        assert t.grad is not None and t.grad.shape == t.shape and torch.isfinite(t.grad.float()).all()


def test_wrong_custom_tensor_count():
    mod = specs.sigmoid_attention(1, 1, 128, 128, 128)
    q = torch.zeros(1, 128, 1, 128, device="cuda", dtype=torch.bfloat16)
    with pytest.raises(TypeError):
        mod(q, q, q)


def _replay_against_eager(run, statics, fresh_inputs, replays=3):
    """Captures run() in a HIP graph, then replays it with new contents in the static input tensors, the program's own
    eager calls and synchronisations between the replays, and compares every replay with the eager result bit for bit."""
    stream = torch.cuda.Stream()
    stream.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(stream):
        for _ in range(2):
            run()                      # warm-up outside capture: first-call set-up (LDS limits, mask analysis) happens here
    torch.cuda.current_stream().wait_stream(stream)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        out = run()
    for i in range(replays):
        for dst, src in zip(statics, fresh_inputs(i)):
            dst.copy_(src)
        graph.replay()
        torch.cuda.synchronize()
        outs = out if isinstance(out, (tuple, list)) else (out,)
        got = [t.clone() for t in outs if t is not None]
        want = run()
        torch.cuda.synchronize()
        want = [t for t in (want if isinstance(want, (tuple, list)) else (want,)) if t is not None]
        for j, (a, b) in enumerate(zip(got, want)):
            assert torch.equal(a, b), f"replay {i}, output {j}"
            assert torch.isfinite(a.float()).all()


def test_operators_replay_in_a_hip_graph():
    """A serving loop captures its step once and replays it: the forward operators (parallel softmax, chunked RetNet, MLA
    decode through its workspace and through the allocation-free entry point) enqueue nothing but kernels on the current
    stream, so a captured call replays to the eager call's bits with new inputs in place."""
    from metaattention_amd import hip_backend as hb
    hb.load_library()
    dev = "cuda"
    # parallel softmax, causal
    B, H, S, D = 1, 4, 384, 128
    mod = specs.softmax_attention(B, H, S, D, D)
    q, k, v = (t.to(dev) for t in inputs.softmax_inputs(B, H, S, D, D, seed=21))
    fresh = lambda i: [t.to(dev) for t in inputs.softmax_inputs(B, H, S, D, D, seed=30 + i)]
    with torch.no_grad():
        _replay_against_eager(lambda: mod(q, k, v), (q, k, v), fresh)
    # chunked RetNet
    Bl, Hl, T, Dk, Dv = 1, 2, 160, 256, 512
    lin = specs.retnet_recurrent(Bl, Hl, T, Dk, Dv)
    gen = lambda seed: [torch.randn(Bl, Hl, T, Dk, generator=torch.Generator().manual_seed(seed)).bfloat16().to(dev),
                        (0.1 * torch.randn(Bl, Hl, T, Dk, generator=torch.Generator().manual_seed(seed + 1))).bfloat16().to(dev),
                        torch.randn(Bl, Hl, T, Dv, generator=torch.Generator().manual_seed(seed + 2)).bfloat16().to(dev)]
    ql, kl, vl = gen(40)
    decay = (1 - torch.exp2(-5 - torch.arange(Hl, dtype=torch.float32)))[None, :, None].expand(Bl, Hl, T).contiguous().to(dev)
    with torch.no_grad():
        _replay_against_eager(lambda: lin(ql, kl, vl, decay), (ql, kl, vl), lambda i: gen(50 + 3 * i))
    # MLA decode with kv splits (workspace from the caching allocator's graph pool) and without any allocation
    Bm, Hq, Skv = 4, 128, 1024
    qm, qpe, kv, kpe = (t.to(dev) for t in inputs.mla_inputs(Bm, Hq, Skv, 512, 64, seed=60))
    fresh_m = lambda i: [t.to(dev) for t in inputs.mla_inputs(Bm, Hq, Skv, 512, 64, seed=61 + i)]
    scale = 576 ** -0.5
    _replay_against_eager(lambda: hb.mla_decode(qm, qpe, kv, kpe, scale=scale, num_split=4), (qm, qpe, kv, kpe), fresh_m)
    out = torch.empty(Bm, 1, Hq, 512, dtype=torch.bfloat16, device=dev)
    _replay_against_eager(lambda: hb.mla_decode(qm, qpe, kv, kpe, scale=scale, num_split=4, out=out, no_alloc=True), (qm, qpe, kv, kpe), fresh_m)


def test_backward_and_decode_operators_replay_in_a_hip_graph():
    """The same for a training step's pieces and the split-KV decode: parallel forward + backward (delta pre-pass, dq and
    dk / dv kernels, workspace from the graph's pool), the chunked backward (three scans and their epilogue kernels) and the
    grouped-query decode with kv splits and per-entry cache lengths."""
    from metaattention_amd import hip_backend as hb
    hb.load_library()
    dev = "cuda"
    B, H, Hkv, S, D, DV = 2, 4, 2, 300, 192, 128
    gen = lambda seed: [torch.randn(B, S, H, D, generator=torch.Generator().manual_seed(seed)).half().to(dev),
                        (0.5 * torch.randn(B, S, Hkv, D, generator=torch.Generator().manual_seed(seed + 1))).half().to(dev),
                        (0.5 * torch.randn(B, S, Hkv, DV, generator=torch.Generator().manual_seed(seed + 2))).half().to(dev),
                        torch.randn(B, S, H, DV, generator=torch.Generator().manual_seed(seed + 3)).half().to(dev)]
    q, k, v, do = gen(100)

    def step():
        lse = torch.empty(B, H, S, device=dev)
        o = hb.attn_fwd(q, k, v, family=hb.MA_ATTN_SOFTMAX, causal=True, scale=D ** -0.5, row_scale=lse)
        return (o, lse) + tuple(hb.attn_bwd(q, k, v, o, do, lse, family=hb.MA_ATTN_SOFTMAX, causal=True, scale=D ** -0.5))
    _replay_against_eager(step, (q, k, v, do), lambda i: gen(110 + 4 * i))

    Bl, Hq, Hl, T, Dk, Dv = 2, 1, 8, 260, 128, 64
    genl = lambda seed: [(0.1 * torch.randn(Bl, Hq, T, Dk, generator=torch.Generator().manual_seed(seed))).bfloat16().to(dev),
                         (0.1 * torch.randn(Bl, Hq, T, Dk, generator=torch.Generator().manual_seed(seed + 1))).bfloat16().to(dev),
                         torch.randn(Bl, Hl, T, Dv, generator=torch.Generator().manual_seed(seed + 2)).bfloat16().to(dev),
                         torch.randn(Bl, Hl, T, Dv, generator=torch.Generator().manual_seed(seed + 3)).bfloat16().to(dev)]
    ql, kl, vl, dol = genl(200)
    ld = torch.nn.functional.logsigmoid(torch.randn(Bl, Hl, T, generator=torch.Generator().manual_seed(7)) + 3.0).to(dev)
    vs = (torch.rand(Bl, Hl, T, generator=torch.Generator().manual_seed(8)) + 0.5).to(dev)
    _replay_against_eager(lambda: hb.linear_bwd(ql, kl, vl, ld, dol, q_scale=1.0, v_scale=vs), (ql, kl, vl, dol), lambda i: genl(210 + 4 * i))

    Bd, G, grp, Sk = 3, 2, 4, 2500
    gend = lambda seed: [torch.randn(Bd, grp, G, 128, generator=torch.Generator().manual_seed(seed)).bfloat16().to(dev),
                         torch.randn(Bd, Sk, G, 128, generator=torch.Generator().manual_seed(seed + 1)).bfloat16().to(dev),
                         torch.randn(Bd, Sk, G, 128, generator=torch.Generator().manual_seed(seed + 2)).bfloat16().to(dev)]
    qd, kd, vd = gend(300)
    lens = torch.tensor([2500, 40, 1999], dtype=torch.int32, device=dev)
    _replay_against_eager(lambda: hb.attn_fwd(qd, kd, vd, family=hb.MA_ATTN_SOFTMAX, causal=False, scale=128 ** -0.5, kv_seqlens=lens),
                          (qd, kd, vd), lambda i: gend(310 + 3 * i))
