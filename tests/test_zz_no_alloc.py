"""ma_mla_decode_noalloc: the entry point that takes no workspace and allocates nothing (the partial results of the kv
splits live in an array inside the library) against ma_mla_decode, through the C ABI."""
import ctypes
import math

import pytest
import torch

from oracle import inputs

pytestmark = pytest.mark.gpu
SCALE = 1 / math.sqrt(576)


def _both(hb, q, q_pe, kv, k_pe, num_split, lens=None):
    """(out, lse) of ma_mla_decode with a workspace tensor, and of ma_mla_decode_noalloc, on the same device tensors."""
    B, _, Hq, D = q.shape
    res = []
    for no_alloc in (False, True):
        out = torch.full((B, 1, Hq, D), float("nan"), dtype=q.dtype, device="cuda")
        lse = torch.full((B, Hq), float("nan"), device="cuda")
        hb.mla_decode(q, q_pe, kv, k_pe, scale=SCALE, num_split=num_split, out=out, lse=lse, kv_seqlens=lens, no_alloc=no_alloc)
        torch.cuda.synchronize()
        res.append((out, lse))
    return res


def test_noalloc_matches_the_workspace_entry_point_twice_in_a_row():
    """Two calls in a row share the scratch array, the second with a smaller input and another split count: both must
    reproduce the existing entry point bit for bit (same kernels, same split), whatever the first call left behind."""
    from metaattention_amd import hip_backend as hb
    hb.load_library()
    for B, Hq, Skv, ns in [(8, 128, 2048, 0), (3, 40, 333, 3), (2, 128, 4096, 8)]:
        q, q_pe, kv, k_pe = (t.cuda() for t in inputs.mla_inputs(B, Hq, Skv, 512, 64, seed=B + Skv))
        (o_ws, lse_ws), (o_na, lse_na) = _both(hb, q, q_pe, kv, k_pe, ns)
        assert torch.isfinite(o_na.float()).all()
        assert torch.equal(o_ws, o_na), (B, Hq, Skv, ns)
        assert torch.equal(lse_ws, lse_na), (B, Hq, Skv, ns)
    # ragged cache lengths with an empty entry, split
    B, Hq, Skv = 4, 128, 640
    q, q_pe, kv, k_pe = (t.cuda() for t in inputs.mla_inputs(B, Hq, Skv, 512, 64, seed=1))
    lens = torch.tensor([Skv, 0, 37, 300], dtype=torch.int32, device="cuda")
    (o_ws, lse_ws), (o_na, lse_na) = _both(hb, q, q_pe, kv, k_pe, 4, lens)
    assert torch.equal(o_ws, o_na) and torch.equal(lse_ws, lse_na)


def test_noalloc_rejects_what_does_not_fit():
    from metaattention_amd import hip_backend as hb
    lib = hb.load_library()
    limit = lib.ma_mla_noalloc_max_workspace()
    assert limit == 40 << 20
    B, Hq, Skv, ns = 64, 128, 4096, 8          # 64 x 8 x 128 x (1024 + 4) bytes = 67 MB of partial results
    q, q_pe, kv, k_pe = (t.cuda() for t in inputs.mla_inputs(B, Hq, Skv, 512, 64, seed=0))
    out = torch.empty(B, 1, Hq, 512, dtype=q.dtype, device="cuda")
    assert hb.mla_workspace_bytes(B, Hq, Skv, num_split=ns) > limit
    with pytest.raises(hb.MetaAttentionError) as ei:
        hb.mla_decode(q, q_pe, kv, k_pe, scale=SCALE, num_split=ns, out=out, no_alloc=True)
    assert ei.value.code == -3 and "scratch" in str(ei.value)
    # the benchmark configuration with the split the library chooses fits
    assert hb.mla_workspace_bytes(B, Hq, Skv) <= limit
    hb.mla_decode(q, q_pe, kv, k_pe, scale=SCALE, out=out, no_alloc=True)
    torch.cuda.synchronize()
    assert torch.isfinite(out.float()).all()
