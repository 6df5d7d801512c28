"""CPU restatement of the paged-MLA work plan (test infrastructure only, see the package docstring).

``mla_work_plan`` follows get_mla_metadata_kernel of the reference
(attention_engine/core/template/cute_template_kvshared/kernels/get_mla_metadata.cu:8-75; host wrapper
flash_api.cpp:25-62): the cache of every batch entry counts ceil(len / block_n) blocks plus a fixed overhead of
``overhead`` blocks; the total is dealt to ``parts`` workers in order, each taking
payload = max(ceil(total / parts) + overhead, 2 * overhead) blocks' worth.  A batch entry that does not fit in what
is left of a worker's payload is cut there (if at least one block fits beside the overhead) and continues on the
next worker as one more split."""
from __future__ import annotations

import numpy as np


def mla_work_plan(seqlens, parts: int, block_n: int = 64, overhead: int = 5):
    """-> (tile_scheduler_metadata int32 [parts, 8], num_splits int32 [B + 1]).
    metadata[p] = (first batch, first token, last batch, end token, split index of the first piece, 0, 0, 0);
    num_splits[b] = number of pieces of the batch entries before b (get_mla_metadata.cu:36-66)."""
    seqlens = [max(int(x), 0) for x in seqlens]
    batch = len(seqlens)
    blocks = [-(-x // block_n) for x in seqlens]
    total = sum(nb + overhead for nb in blocks)
    payload = max(-(-total // parts) + overhead, 2 * overhead)
    meta = np.zeros((parts, 8), dtype=np.int32)
    splits = np.zeros(batch + 1, dtype=np.int32)
    now_idx = now_block = now_split = cum = 0
    for p in range(parts):
        meta[p, 0], meta[p, 1], meta[p, 4] = now_idx, now_block * block_n, now_split
        remain = payload
        while now_idx < batch:
            left = blocks[now_idx] - now_block
            if remain >= left + overhead:
                cum += now_split + 1
                splits[now_idx + 1] = cum
                remain -= left + overhead
                now_idx += 1
                now_block = now_split = 0
            else:
                if remain - overhead > 0:
                    now_block += remain - overhead
                    now_split += 1
                    remain = 0
                break
        meta[p, 2] = now_idx if now_block > 0 else now_idx - 1
        meta[p, 3] = now_block * block_n if now_block > 0 else (seqlens[now_idx - 1] if now_idx > 0 else 0)
    assert now_idx == batch and now_block == 0 and now_split == 0, "the plan must consume every batch entry (get_mla_metadata.cu:68)"
    return meta, splits


def plan_pieces(meta, splits, seqlens):
    """The (batch, begin token, end token, split index) pieces a plan hands out, part by part, as the split kernel of
    the reference walks them (kernels/splitkv_mla.cu:1127-1150): the first piece of a part starts at its metadata's
    first token with its split index, later pieces at token 0 with split index 0; the last piece ends at the
    metadata's end token, earlier ones at their batch entry's length."""
    out = []
    batch = len(seqlens)
    for p in range(meta.shape[0]):
        b0, t0, b1, t1, s0 = (int(x) for x in meta[p, :5])
        if b0 >= batch:
            continue
        for b in range(b0, b1 + 1):
            begin = t0 if b == b0 else 0
            end = min(t1 if b == b1 else max(int(seqlens[b]), 0), max(int(seqlens[b]), 0))
            out.append((p, b, begin, end, s0 if b == b0 else 0))
    return out
