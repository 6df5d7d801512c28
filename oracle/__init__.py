"""CPU oracle for the attention forward hot path.

TEST INFRASTRUCTURE ONLY.  Nothing in the shipped package imports this
directory: it is used by ``tests/``, by ``__graft_entry__.smoke()`` and by the
``cpu_baseline`` leg of ``bench.py`` as the checker / the timed CPU baseline,
never as the thing measured or shipped.

Every function restates, in plain fp32/fp64 PyTorch on the CPU, one of the
inline PyTorch reference functions that the reference repository's own test
script compares its kernels against (each docstring cites the file:line it
follows).  The reference holds no golden vectors for this path, so each
restatement is pinned by independent checks in ``tests/test_oracle.py``:

=====================  =====================================================
function               pinned by
=====================  =====================================================
softmax_attention      torch SDPA / logsumexp in fp64, closed forms (constant
                       K gives running mean of V; S=1 gives O=V), brute force
sigmoid_attention      element-wise closed form 1/(1+exp(-x)) brute force;
                       masked entries contribute exactly 0
relu_attention         brute-force loops on tiny shapes
retention_parallel     brute force fp64; clamp invariant (rows with
                       sum|.|<1 stay un-normalised); all-ones mask special case;
                       freeze_r (the gradient with the row scale held constant):
                       autograd == the written-out dq, dk, dv; == the true
                       gradient where the clamp holds r at 1
retnet_chunked         3-way agreement: quadratic form == token recurrence
                       == chunked form for several chunk sizes (fp64)
ssd_chunk_scan         3-way agreement: chunked reference == naive sequential
                       state-space recurrence; chunk-size independence
simple_gla             token-by-token recurrence (fp64)
mla_decode             SDPA with K=concat(kv,k_pe), V=kv; split-KV invariance
sparse_decode_attention  dense attention over the gathered kept keys only
paged_mla_decode       mla_decode on the contiguous cache (identity table); invariance
                       to a permutation of the page pool
mla_work_plan          hand-computed small plans; invariants on random ragged batches:
                       the pieces tile every batch entry exactly once in order, piece
                       counts equal num_splits, no part exceeds its payload
masked_attention       SDPA with a boolean attn_mask (fp64); tril keep mask ==
                       softmax_attention(causal); a block mask == attention over
                       the gathered kept keys of each query block; rows without
                       keys are 0; sigmoid / relu by element-wise brute force
biased_attention       SDPA with a float attn_mask (fp64), with and without the causal
                       triangle; add = 0 == softmax_attention; a seq_len_kv vector equal for
                       all keys leaves softmax unchanged and shifts lse by it; soft-capping,
                       sigmoid and relu element by element
attention_grads,       central differences of the pinned forward functions in
linear_attention_grads fp64 along random directions; SDPA's own autograd
(all of the above)     tests/golden/*.npz: the operators' definitions evaluated
                       element by element in fp64 numpy by independent code
=====================  =====================================================

No function here is "parity unpinned".
"""
from .attention_ref import (  # noqa: F401
    softmax_attention,
    sigmoid_attention,
    relu_attention,
    retention_parallel,
    mla_decode,
    retention_decay_mask,
    attention_grads,
    sparse_decode_attention,
    paged_mla_decode,
    masked_attention,
    biased_attention,
)
from .linear_ref import (  # noqa: F401
    retnet_quadratic,
    retnet_recurrence,
    linear_attention_chunked,
    ssd_chunk_scan_combined,
    ssd_sequential,
    simple_gla_chunked,
    simple_gla_recurrence,
    linear_attention_grads,
)
from .mla_plan_ref import mla_work_plan, plan_pieces  # noqa: F401
from .compare import assert_close, mismatch_report  # noqa: F401
from . import inputs  # noqa: F401
