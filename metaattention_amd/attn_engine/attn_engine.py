"""``AttentionEngine`` / ``OnlineFunc``: the public spec API of the parallel,
decode and MLA operators (attention_engine/attn_engine/attn_engine.py:16-408),
backed by the pre-built gfx950 kernel library instead of run-time code
generation.

Construction traces the user's spec, canonicalises it (core/canonical.py) and
picks a kernel variant; nothing is compiled, tuned or cached on disk.  The
call takes GPU tensors in the reference's layouts and enqueues the kernels on
the current stream.
"""
from __future__ import annotations

import math
import weakref

import torch

from core.canonical import canonicalize_score_mod, classify_mask, identify_online_func
from core.transform.core import CustomIO, SymbolicArray, SymbolScalar, Var
from autotuner.arch import MI355X


class OnlineFunc:
    """Row function of an online (tiled) attention forward.

    ``online_rowscales``: running per-row statistics, each a
    ``SymbolScalar(name, Var(init))`` with init "-inf", "0.0" or "1";
    ``final_rowscales``: what is kept after the last tile.
    ``online_fwd(scores, online_rowscales, b, h, q_idx)`` returns
    ``(scores', online_rowscales', o_scale)``: the probabilities of this tile,
    the updated statistics and the factor the output accumulator is rescaled
    by.  ``online_fwd_epilogue(o, online_rowscales, b, h, q_idx)`` returns
    ``(o', final_rowscales)``.  ``forward`` / ``backward`` describe the
    recompute for a backward pass and ``combine`` the split-KV merge.  The
    kernel library holds one version of each per row function; where a spec
    overrides them, its traced version is compared with the library's and a
    spec that computes something else is refused (core/canonical.py).
    """

    def __init__(self, online_rowscales: dict, final_rowscales: dict, external_fwd_tensors: CustomIO):
        self.online_rowscales = online_rowscales
        self.final_rowscales = final_rowscales
        self.vars = {"scores": SymbolicArray(), "o_scale": None}
        self.external_fwd_tensors = external_fwd_tensors
        self.doosum_rowscales = SymbolicArray("doosum", Var("doosum"), shape_idx=["block_M"])

    @staticmethod
    def online_fwd(scores, online_rowscales, b, h, q_idx):
        return scores, online_rowscales, SymbolScalar("o_scale", Var("o_scale"))

    @staticmethod
    def online_fwd_epilogue(o, online_rowscales, b, h, q_idx):
        return o, online_rowscales

    @staticmethod
    def forward(scores, final_rowscales, b, h, q_idx, kv_idx):
        return scores

    @staticmethod
    def backward(dp, scores, final_rowscales, b, h, q_idx, kv_idx):
        return dp

    @staticmethod
    def combine(final_rowscales):
        return SymbolScalar("o_scale", Var("o_scale"))


_FAMILY = {
    ("identity", "softmax"): "softmax",
    ("sigmoid", "identity"): "sigmoid",
    ("relu", "identity"): "relu",
    ("identity", "retention"): "retention",
}


def _kernel_view(t):
    """t itself when the kernels can read it in place, else a contiguous copy (gradients flow through the copy)."""
    ok = t.stride(-1) == 1 and t.data_ptr() % 16 == 0 and all(s % 8 == 0 for s in t.stride()[:-1])
    return t if ok else t.contiguous()


class _ForwardOnly(torch.autograd.Function):
    """Gives outputs a grad_fn whose backward fails loudly, for the operators whose
    backward kernels are not in the library."""

    @staticmethod
    def forward(ctx, run, *tensors):
        return run(*tensors)

    @staticmethod
    def backward(ctx, *grads):
        raise NotImplementedError("this operator is forward-only: its backward kernel is not part of the gfx950 kernel library")


class _Attention(torch.autograd.Function):
    """Forward + backward of the softmax / sigmoid / relu / retention operators, as _attention of
    tl_template/attn/attn_tl.py:654-692: saves q, k, v, o and the final row scale, returns
    (dq, dk, dv) and None for every custom input."""

    @staticmethod
    def forward(ctx, engine, run, fam_code, bias_t, call_masks, score_mask, extras, q, k, v):
        out = run(q, k, v)
        lse = engine.final_rowscales
        ctx.engine, ctx.fam_code, ctx.bias_t, ctx.call_masks, ctx.score_mask = engine, fam_code, bias_t, call_masks, score_mask
        ctx.extras = extras
        ctx.save_for_backward(q, k, v, out, *([lse] if lse is not None else []))
        return out

    @staticmethod
    def backward(ctx, dout):
        from hip_backend import attn_bwd
        q, k, v, out, *rest = ctx.saved_tensors
        form = ctx.engine.score_form
        eng = ctx.engine
        masks, causal = {}, eng.mask_kind == "causal"
        if ctx.call_masks is not None:
            # a call with an external block mask: the whole mask (the caller's blocks, the mask_mod, causal) as elements
            masks, causal = ctx.call_masks(), False
        elif eng.mask_kind.startswith("other"):
            masks = dict(zip(("elem_mask", "elem_mask_t", "kv_block_mask", "q_block_mask"),
                             eng._dense_mask(q.shape[0], q.shape[2], q.shape[1], k.shape[1], q.device, transposed=True)))
        if ctx.score_mask is not None:
            # retention: the multiplier tensor in both orientations (the dk / dv kernels walk down its columns)
            masks = dict(score_mask=ctx.score_mask, score_mask_t=ctx.score_mask.transpose(2, 3).contiguous())
        dq, dk, dv = attn_bwd(q, k, v, out, dout, rest[0] if rest else None, family=ctx.fam_code,
                              causal=causal, scale=form.scale, bias=form.bias, bias_tensor=ctx.bias_t, **masks, **ctx.extras)
        return None, None, None, None, None, None, None, dq, dk, dv


class AttentionEngine:
    def __init__(self, qkv_meta, custom_fwd_inputs, score_mod, mask_mod, online_func,
                 mask_value="-inf", device=None, backend="tl",
                 tune=False, tune_file="", tune_bwd=False, tune_file_bwd="",
                 infer_mask=True, infer_mask_block_M=128, infer_mask_block_N=128,
                 extern_block_mask=False, use_varlen=False, kv_shared=False):
        # `backend`, `tune*`, `infer_mask*` select code generators / tuners in the
        # reference; here there is one pre-built backend and fixed tile tables, so
        # they are accepted and ignored, except infer_mask_block_N: the block size of an
        # external kv block mask (examples/sparse_gqa_decode.py:100-107).
        self.device = device if device is not None else MI355X()
        self.use_varlen = use_varlen
        self.block_mask = None
        self.tl_code = ""     # no source is generated
        self.extern_block_mask = extern_block_mask
        self.kv_block_size = int(infer_mask_block_N)
        self._infer_blocks = (int(infer_mask_block_M), int(infer_mask_block_N)) if infer_mask else None
        if (use_varlen or extern_block_mask) and (self.kv_block_size < 32 or self.kv_block_size % 32 != 0):
            raise NotImplementedError("kv block masks need a block size that is a multiple of 32 (infer_mask_block_N)")
        if (use_varlen or extern_block_mask) and kv_shared:
            raise NotImplementedError("varlen / external block masks are not in the MLA decode operator")
        if use_varlen and qkv_meta[0].shape[2] == qkv_meta[2].shape[2]:
            raise NotImplementedError("cache lengths (use_varlen) are only in the decode operators of the kernel library")
        dtype = qkv_meta[0].dtype
        if dtype not in (torch.float16, torch.bfloat16):
            raise KeyError(dtype)      # the reference's dtype map has only these two (attn_engine.py:234-237)
        self.dtype = dtype
        B, Hq, Sq, Dqk = qkv_meta[0].shape
        Hkv, Skv, Dv = qkv_meta[2].shape[1], qkv_meta[2].shape[2], qkv_meta[2].shape[3]
        self.meta = dict(B=B, Hq=Hq, Hkv=Hkv, Sq=Sq, Skv=Skv, Dqk=Dqk, Dv=Dv)
        self.custom_fwd_inputs = custom_fwd_inputs if custom_fwd_inputs is not None else CustomIO()

        # dispatch by shape, as attn_engine.py:227-343
        if kv_shared:
            self._init_mla(backend)
        elif Hq % Hkv != 0:
            raise NotImplementedError("heads of q must be a multiple of the heads of k and v")
        else:
            # prefill, multi-head or grouped-query (attn_engine.py:305-343: same kernel family, kv head = head // groups).
            # Dense decode (seq_len_q != seq_len_kv, attn_engine.py:262-303; the examples pad the declared seq_len_q to
            # a multiple of 128 and pass the real query, examples/mha_decode.py:104-108) runs through the same kernels
            # with no structural mask; the reference's split-KV launch and its block-sparse variants have no counterpart.
            self._init_prefill(score_mod, mask_mod, online_func, mask_value)

    # ------------------------------------------------------------------ prefill
    def _init_prefill(self, score_mod, mask_mod, online_func, mask_value):
        m = self.meta
        form = canonicalize_score_mod(score_mod, self.custom_fwd_inputs)
        row, inner = identify_online_func(online_func, return_scale=True)
        if inner != 1.0:
            # a softmax that scales the scores itself (examples/mha_v2.py:44-69): the library's softmax of inner * score
            if form.activation != "identity" or form.bias_tensor or form.mask_tensor or form.extra or form.softcap is not None:
                raise NotImplementedError("an OnlineFunc that scales the scores itself goes with a score_mod of the form a * score + c")
            form.scale, form.bias = form.scale * inner, form.bias * inner
        fam = _FAMILY.get((form.activation, row))
        if fam is None:
            raise NotImplementedError(f"no library kernel for score activation '{form.activation}' with row function '{row}'")
        if fam == "retention" and form.mask_tensor is None:
            raise NotImplementedError("retention row function without an element-wise score multiplier tensor")
        if fam != "retention" and form.mask_tensor is not None:
            raise NotImplementedError("element-wise score multiplier tensors are only in the retention kernel")
        if not form.scale > 0:
            raise NotImplementedError("score scale must be positive")
        if mask_value not in ("-inf", "0"):
            raise NotImplementedError(f"mask_value {mask_value!r}")
        self.mask_kind = classify_mask(mask_mod, m["B"], m["Hq"], m["Sq"], m["Skv"])
        self.mask_mod, self._mask_tensors = mask_mod, None
        if self.mask_kind.startswith("other"):
            # any other mask_mod: evaluated densely once (the reference does the same to infer its block mask,
            # lower.py:723-740) into an element-wise keep mask plus a block mask for tile skipping
            if fam == "retention":
                raise NotImplementedError("the retention kernel takes the causal structural mask or none")
            if m["Sq"] != m["Skv"] and m["Sq"] % 128 != 0:
                pass     # (a declared query length padded for decode: the mask is built for the tensors actually passed)
            dense_bytes = (m["B"] * m["Hq"] if self.mask_kind == "other_bh" else 1) * m["Sq"] * m["Skv"]
            if dense_bytes > 2 ** 31:
                raise NotImplementedError("a mask_mod that depends on batch or head at this size needs more than 2 GiB as a dense mask")
        # mask_value "0": the reference applies no element-wise mask in forward, only causal
        # tile skipping (lower.py:638, attn_tl.py:140-151); the retention kernel does the same.
        if mask_value == "0" and fam != "retention" and self.mask_kind != "none":
            raise NotImplementedError("mask_value '0' is only in the retention kernel")
        self.family, self.score_form = fam, form
        self.names = list(self.custom_fwd_inputs.input_tensors)
        self.final_rowscales = None
        self.attention = self._call_prefill

    def _call_prefill(self, q, k, v, *custom, block_mask=None, cache_seqlens=None):
        from hip_backend import attn_fwd, MA_ATTN_SOFTMAX, MA_ATTN_SIGMOID, MA_ATTN_RELU, MA_ATTN_RETENTION
        fam_code = {"softmax": MA_ATTN_SOFTMAX, "sigmoid": MA_ATTN_SIGMOID, "relu": MA_ATTN_RELU,
                    "retention": MA_ATTN_RETENTION}[self.family]
        if len(custom) != len(self.names):
            raise TypeError(f"expected {len(self.names)} custom tensor(s) {self.names} after q, k, v; got {len(custom)}")
        given = dict(zip(self.names, custom))
        form = self.score_form

        # block_mask [batch, heads, q blocks, kv blocks]: the block-sparse prefill operator (blockattn_tl.py:123-234);
        # [batch, heads_kv, kv blocks] (+ cache_seqlens): the varlen block-sparse decode operator
        prefill_blocks = block_mask if block_mask is not None and block_mask.dim() == 4 else None
        if prefill_blocks is not None:
            block_mask = None
            if self.family == "retention" or cache_seqlens is not None:
                raise NotImplementedError("block-sparse prefill masks go with the softmax / sigmoid / relu kernels, without cache_seqlens")
        sparse = block_mask is not None or cache_seqlens is not None
        if sparse and (self.mask_kind != "none" or self.family == "retention"):
            raise NotImplementedError("block_mask / cache_seqlens are for the unmasked decode operators")
        if block_mask is not None and block_mask.dim() != 3:
            raise NotImplementedError("block masks are [batch, heads_kv, kv blocks] (decode) or [batch, heads, q blocks, kv blocks] (prefill)")

        # (decided here: inside an autograd function's forward, gradient mode is off)
        needs_grad = torch.is_grad_enabled() and any(t.requires_grad for t in (q, k, v))
        # the kernels read strided views in place (rows of 16-byte aligned, 16-byte multiples); any other view is copied once,
        # as a caller of the reference's operator would have to (its kernels take contiguous tensors: attn_tl.py:69-70)
        q, k, v = (_kernel_view(t) for t in (q, k, v))

        def run(q, k, v):
            B, Sq, H, D = q.shape
            Hkv, Dv = k.shape[2], v.shape[-1]
            grp = H // Hkv
            kw = dict(family=fam_code, causal=self.mask_kind == "causal", scale=form.scale, bias=form.bias,
                      bias_tensor=given[form.bias_tensor].to(torch.float32) if form.bias_tensor else None)
            kw.update(self._additive_inputs(given, H, q.dtype, q.device))
            if self.mask_kind.startswith("other"):
                elem, _ = self._dense_mask(B, H, Sq, k.shape[1], q.device)
                # (block entries 0 / 1 / 2: nothing, something, everything kept; the kernels skip the 0s and do not read
                # the element mask for the 2s)
                kw.update(elem_mask=elem, kv_block_mask=self._mask_tensors[4], kv_block_size=32)
            if prefill_blocks is not None:
                ext = self._expand_block_mask(prefill_blocks, B, H, Sq, k.shape[1])
                if "kv_block_mask" in kw:
                    ext = ext * kw["kv_block_mask"]        # (the mask_mod's own block mask: broadcast over batch / heads)
                kw.update(kv_block_mask=ext.contiguous(), kv_block_size=32)
            if sparse:
                kw.update(kv_seqlens=cache_seqlens.to(torch.int32) if cache_seqlens is not None else None, kv_block_mask=block_mask,
                          kv_block_size=self.kv_block_size if block_mask is not None else 0)
            has_rs = self.family in ("softmax", "retention")
            if Sq == 1 and grp > 1 and self.mask_kind == "none" and self.family != "retention":
                # one query token, grouped-query: the query heads of a kv head become the rows of that head
                # (the decode kernels of the reference pack them the same way, attn_gqa_decode_tl.py:81-84)
                out = torch.empty(B, 1, H, Dv, dtype=q.dtype, device=q.device)
                rs = torch.empty(B, Hkv, grp, dtype=torch.float32, device=q.device) if has_rs else None
                attn_fwd(q.contiguous().view(B, Hkv, grp, D).transpose(1, 2), k, v, out=out.view(B, Hkv, grp, Dv).transpose(1, 2),
                         row_scale=rs, **kw)
                self.final_rowscales = rs.view(B, H, 1) if has_rs else None
                return out
            rs = torch.empty(B, H, Sq, dtype=torch.float32, device=q.device) if has_rs else None
            mask_t = given[form.mask_tensor] if form.mask_tensor else None
            if mask_t is not None and mask_t.dtype != q.dtype:
                mask_t = mask_t.to(q.dtype)
            gamma = None
            if (mask_t is not None and self.family == "retention" and kw["causal"] and (D, Dv) == (256, 512) and Sq == k.shape[1]
                    and not needs_grad):
                gamma = self._decay_gamma_of(given[form.mask_tensor], H, Sq)
            self.last_call_generated_mask = gamma is not None     # (which of the two forms the last call took)
            if gamma is not None:
                # the multiplier is gamma_h^(i - j) [i >= j]: the kernel generates it instead of reading the tensor once per
                # batch entry and column half (the row function sees fp32 factors where the tensor holds rounded ones)
                out = attn_fwd(q, k, v, decay_gamma=gamma, row_scale=rs, **kw)
            else:
                out = attn_fwd(q, k, v, score_mask=mask_t, row_scale=rs, **kw)
            self.final_rowscales = rs     # kept for a backward pass, not returned (attn_tl.py:661-667)
            return out

        if sparse:
            # the varlen block-sparse decode operator squeezes the query token and has no backward
            # (blockattn_decode_varlen_tl.py:17, :250)
            return run(q, k, v).squeeze(1)

        if any(t.requires_grad for t in (q, k, v)):
            extras = {}
            if form.extra or form.softcap is not None:
                # the backward kernels recompute the score with its additive terms and soft-capping (the custom inputs
                # themselves get no gradient, as in the reference, attn_tl.py:692)
                if self.family == "retention":
                    return _ForwardOnly.apply(run, q, k, v)
                extras = self._additive_inputs(given, q.shape[2], q.dtype, q.device)
            score_mask = None
            if self.family == "retention":
                # head sizes the backward kernels of the retention operator are built for (256 / 512 is its own,
                # examples/retention_parallel.py)
                if (q.shape[-1], v.shape[-1]) not in ((256, 512), (128, 128), (64, 64), (128, 256), (256, 256)) or not form.mask_tensor:
                    return _ForwardOnly.apply(run, q, k, v)
                score_mask = given[form.mask_tensor]
                score_mask = score_mask if score_mask.dtype == q.dtype else score_mask.to(q.dtype)
            bias_t = given[form.bias_tensor].to(torch.float32) if form.bias_tensor else None
            call_masks = None
            if prefill_blocks is not None:
                shape = (q.shape[0], q.shape[2], q.shape[1], k.shape[1], q.device)
                call_masks = lambda: self._block_mask_backward_masks(prefill_blocks, *shape)
            return _Attention.apply(self, run, fam_code, bias_t, call_masks, score_mask, extras, q, k, v)
        return run(q, k, v)

    def _additive_inputs(self, given, H, dtype, device):
        """The score_mod's score-free terms as the kernel takes them: one tensor addressed [b, h, q, kv] with strides
        (a single custom tensor is passed as it is, through a broadcasting view; several are summed once per call),
        per-head slopes for the terms in q_idx / kv_idx, and the soft-capping constant."""
        from core.eager import custom_tensor_view
        form = self.score_form
        kw = {}
        if form.softcap is not None:
            kw["softcap"] = form.softcap
        syms = self.custom_fwd_inputs.input_tensors
        adds, slopes = [], {"q_idx": None, "kv_idx": None}
        for mono, coef in form.extra.items():
            idx = [f[2:] for f in mono if f.startswith("i:")]
            tens = [f[2:] for f in mono if not f.startswith("i:")]
            if idx:
                sl = torch.full((H,), float(coef), dtype=torch.float32, device=device)
                if tens:
                    sl = sl * given[tens[0]].to(torch.float32).reshape(-1).expand(H) if given[tens[0]].numel() in (1, H) else None
                    if sl is None:
                        raise ValueError(f"custom tensor '{tens[0]}' multiplying {idx[0]} must have one element or one per head")
                slopes[idx[0]] = sl if slopes[idx[0]] is None else slopes[idx[0]] + sl
            else:
                adds.append((coef, custom_tensor_view(given[tens[0]], syms[tens[0]].shape_idx)))
        if len(adds) == 1 and adds[0][0] == 1.0 and adds[0][1].dtype in (torch.float32, dtype):
            kw["score_add"] = adds[0][1]
        elif adds:
            total = None
            for coef, t in adds:
                term = t.to(torch.float32) * coef
                total = term if total is None else total + term
            kw["score_add"] = total
        if slopes["q_idx"] is not None:
            kw["pos_slope_q"] = slopes["q_idx"].contiguous()
        if slopes["kv_idx"] is not None:
            kw["pos_slope_kv"] = slopes["kv_idx"].contiguous()
        return kw

    @staticmethod
    def _expand_block_mask(block_mask, B, H, Sq, Skv):
        """A caller's block mask [1|B, 1|H, nq, nk] (non-zero = keep; a block covers Sq/nq query rows and Skv/nk keys,
        blockattn_tl.py:109-112, :170) at the kernel's granularity: uint8 [.., Sq/128, Skv/32]."""
        if block_mask.shape[0] not in (1, B) or block_mask.shape[1] not in (1, H):
            raise ValueError(f"block_mask {tuple(block_mask.shape)} does not fit batch {B}, heads {H}")
        nq, nk = block_mask.shape[2:]
        if nq < 1 or nk < 1 or Sq % nq or Skv % nk or (Sq // nq) % 128 or (Skv // nk) % 32:
            raise NotImplementedError(f"block_mask of {nq} x {nk} blocks over {Sq} x {Skv}: blocks must be a whole multiple of "
                                      "128 query rows by 32 keys")
        keep = (block_mask != 0).to(torch.uint8)
        return keep.repeat_interleave(Sq // nq // 128, dim=2).repeat_interleave(Skv // nk // 32, dim=3)

    def _block_mask_backward_masks(self, block_mask, B, H, Sq, Skv, device):
        """The masks the backward kernels take, for a call with an external block mask: the caller's blocks spread to
        elements and ANDed with the operator's own mask (the mask_mod, or causal), its transpose, and both pooled to the
        blocks the kernels skip by.  Built per backward call (the block mask is an argument of the call, not of the
        operator); 2 x batch x heads x Sq x Skv bytes unless the mask broadcasts."""
        nq, nk = block_mask.shape[2:]
        elem = (block_mask != 0).repeat_interleave(Sq // nq, dim=2).repeat_interleave(Skv // nk, dim=3)
        if self.mask_kind == "causal":
            elem = elem & torch.ones(Sq, Skv, dtype=torch.bool, device=device).tril_()
        elif self.mask_kind.startswith("other"):
            elem = elem & (self._dense_mask(B, H, Sq, Skv, device)[0] != 0)
        Bm, Hm = elem.shape[:2]
        elem_t = elem.transpose(2, 3)

        def pool(m, r, c):                        # blocks of 128 rows x 32 columns: 0 nothing kept, 1 some, 2 every element
            rp = (r + 127) // 128 * 128
            m = torch.nn.functional.pad(m, (0, 0, 0, rp - r)) if rp != r else m
            m = m.reshape(Bm, Hm, rp // 128, 128, c // 32, 32)
            return (m.any(dim=5).any(dim=3).to(torch.uint8) + m.all(dim=5).all(dim=3).to(torch.uint8)).contiguous()

        return dict(elem_mask=elem.to(torch.uint8).contiguous(), elem_mask_t=elem_t.to(torch.uint8).contiguous(),
                    kv_block_mask=pool(elem, Sq, Skv), q_block_mask=pool(elem_t, Skv, Sq))

    def _dense_mask(self, B, H, Sq, Skv, device, transposed=False):
        """(element-wise keep mask uint8 [1|B, 1|H, Sq, Skv] with 4-byte aligned rows, block mask uint8
        [1|B, 1|H, ceil(Sq/128), ceil(Skv/32)]: a block is kept when any of its elements is) for the mask_mod, built
        once per shape on the device.  transposed=True: (the keep mask, its transpose [.., Skv, Sq] with 4-byte aligned
        rows, the block mask, the block mask of the transpose [.., ceil(Skv/128), ceil(Sq/32)]) for the backward kernels;
        the transposed pair is built on first use."""
        from core.transform.core import create_mask
        key = (B, H, Sq, Skv, str(device))
        if self._mask_tensors is None or self._mask_tensors[0] != key:
            Bm, Hm = (B, H) if self.mask_kind == "other_bh" else (1, 1)
            dense = create_mask(self.mask_mod, Bm, Hm, Sq, Skv, device)
            skp, sqp, nkp = (Skv + 3) // 4 * 4, (Sq + 127) // 128 * 128, (Skv + 31) // 32 * 32
            buf = torch.zeros(Bm, Hm, Sq, skp, dtype=torch.uint8, device=device)
            buf[..., :Skv] = dense
            pad = torch.zeros(Bm, Hm, sqp, nkp, dtype=torch.bool, device=device)
            pad[:, :, :Sq, :Skv] = dense
            tiles = pad.view(Bm, Hm, sqp // 128, 128, nkp // 32, 32)
            blocks = tiles.any(dim=5).any(dim=3).to(torch.uint8).contiguous()
            # for the backward kernels: 2 where the mask keeps every element of the tile (it is then not consulted there)
            blocks_bwd = (blocks + tiles.all(dim=5).all(dim=3).to(torch.uint8)).contiguous()
            self._mask_tensors = [key, buf[..., :Skv], blocks, None, blocks_bwd]
            if self._infer_blocks is not None:
                # the attribute the reference keeps for operators whose mask is not the exact causal one
                # (attn_engine.py:394-397): the mask_mod pooled to infer_mask_block_M x infer_mask_block_N blocks
                bm_, bn_ = self._infer_blocks
                qp, kp = (Sq + bm_ - 1) // bm_ * bm_, (Skv + bn_ - 1) // bn_ * bn_
                padb = torch.zeros(Bm, Hm, qp, kp, dtype=torch.bool, device=device)
                padb[:, :, :Sq, :Skv] = dense
                self.block_mask = padb.view(Bm, Hm, qp // bm_, bm_, kp // bn_, bn_).any(dim=5).any(dim=3).to(torch.int8)
        if transposed:
            if self._mask_tensors[3] is None:
                elem = self._mask_tensors[1]
                buf_t = torch.zeros(elem.shape[0], elem.shape[1], Skv, (Sq + 3) // 4 * 4, dtype=torch.uint8, device=device)
                buf_t[..., :Sq] = elem.transpose(2, 3)
                skp, sqp = (Skv + 127) // 128 * 128, (Sq + 31) // 32 * 32
                pad = torch.zeros(elem.shape[0], elem.shape[1], skp, sqp, dtype=torch.bool, device=device)
                pad[:, :, :Skv, :Sq] = elem.transpose(2, 3) != 0
                tiles_t = pad.view(elem.shape[0], elem.shape[1], skp // 128, 128, sqp // 32, 32)
                blocks_t = tiles_t.any(dim=5).any(dim=3).to(torch.uint8) + tiles_t.all(dim=5).all(dim=3).to(torch.uint8)
                self._mask_tensors[3] = (buf_t[..., :Sq], blocks_t.contiguous())
            return self._mask_tensors[1], self._mask_tensors[3][0], self._mask_tensors[4], self._mask_tensors[3][1]
        return self._mask_tensors[1], self._mask_tensors[2]

    # ------------------------------------------------------------------ MLA decode
    def _init_mla(self, backend="tl"):
        m = self.meta
        if m["Hkv"] != 1:
            raise AssertionError("MLA decode needs a single latent kv head")   # mla_decode_tl.py:58
        if m["Sq"] != 1:
            raise NotImplementedError("MLA decode takes one query token")
        self.mla_dim, self.mla_pe = m["Dv"], m["Dqk"] - m["Dv"]
        # the spec's score_mod / online_func are not consumed on this path
        # (core/lower/lower_decode_mla.py:25-38): fixed softmax, scale (d + d_pe)^-0.5
        self.mla_scale = 1.0 / math.sqrt(m["Dqk"])
        self.attention = self._call_mla
        if backend in ("cute", "cute_v2"):
            # the paged interface of the reference's second MLA backend (attn_engine.py:196-224): mod(q [B,1,Hq,576],
            # k_cache [B * Skv / 64, 64, 1, 576]) -> (out, lse), every sequence full, pages in order
            self.attention = self._call_mla_paged

    def _decay_gamma_of(self, mask, H, S):
        """fp32 [H] gamma if the retention operator's multiplier tensor `mask` [1, H, S, S] is a per-head exponential decay
        gamma_h^(i - j) for j <= i (whatever lies above the diagonal is never read under the causal mask), else None.
        Decided on the device, once per tensor object and version counter: log2 gamma_h is fitted to the first
        column, the whole lower triangle is then compared with the regenerated mask to two units in the last place of the
        tensor's dtype.  examples/retention_parallel.py:25-111 builds exactly such a mask."""
        # (remembered per tensor OBJECT and version counter: an address alone could be a new tensor in recycled memory)
        cache = self.__dict__.setdefault("_gamma_cache", [])
        for ref, version, known in cache:
            if ref() is mask and version == mask._version:
                return known
        gamma = None
        if mask.dim() == 4 and tuple(mask.shape) == (1, H, S, S) and S >= 2:
            col = mask[0, :, :, 0].float()                              # [H, S]: gamma_h^i
            i = torch.arange(S, device=mask.device, dtype=torch.float32)
            ok = col > 1e-30
            lg = torch.log2(col.clamp_min(1e-30))
            w = torch.where(ok, i, torch.zeros_like(i))                 # least squares through the origin: sum i lg / sum i^2
            l2g = (w * lg).sum(dim=1) / (w * i).sum(dim=1).clamp_min(1.0)
            if bool(ok[:, :2].all()) and bool((l2g <= 0).all()) and bool(torch.isfinite(l2g).all()):
                diff = (i.view(S, 1) - i.view(1, S)).clamp_min(0.0)
                lower = i.view(S, 1) >= i.view(1, S)
                eps = 2.0 ** (-7 if mask.dtype == torch.bfloat16 else -10)    # two units in the last place
                same = torch.ones((), dtype=torch.bool, device=mask.device)
                for h in range(H):                                      # (head by head: fp32 temporaries of one [S, S] plane, not of H)
                    want = torch.exp2(diff * l2g[h])
                    same &= (((mask[0, h].float() - want).abs() <= eps * want + 1e-30) | ~lower).all()
                if bool(same):
                    gamma = torch.exp2(l2g).contiguous()
        cache[:] = [e for e in cache if e[0]() is not None and e[0]() is not mask][-7:]
        cache.append((weakref.ref(mask), mask._version, gamma))
        return gamma

    def _call_mla_paged(self, q, k_cache):
        from hip_backend import flash_mla_with_kvcache
        m = self.meta
        page = k_cache.shape[1]
        # The reference's table (attn_engine.py:211-216): sequence b owns pages b * pad / page .. of the pool, where pad is
        # the cache length rounded up to 256, so the pool must hold B * pad / page pages.
        pad = ((m["Skv"] + 255) // 256) * 256
        if pad % page != 0 or k_cache.shape[0] < m["B"] * pad // page:
            raise ValueError(f"paged MLA cache: expected a pool of at least {m['B']} x {pad} / {page} pages of {page} rows (cache length "
                             f"{m['Skv']} rounded up to 256, as the reference lays it out), got {tuple(k_cache.shape)}")
        table = torch.arange(m["B"] * pad // page, dtype=torch.int32, device=q.device).view(m["B"], pad // page)
        lens = torch.full((m["B"],), m["Skv"], dtype=torch.int32, device=q.device)
        return flash_mla_with_kvcache(q, k_cache, table, lens, m["Dv"], softmax_scale=self.mla_scale)

    def _call_mla(self, q, q_pe, kv, k_pe):
        from hip_backend import mla_decode
        return mla_decode(*(_kernel_view(t) for t in (q, q_pe, kv, k_pe)), scale=self.mla_scale)

    def __call__(self, *args, **kargs):
        block_mask, cache_seqlens = kargs.get("block_mask"), kargs.get("cache_seqlens")
        if block_mask is None and cache_seqlens is None:
            return self.attention(*args)
        if self.attention != self._call_prefill:
            raise NotImplementedError("block_mask / cache_seqlens are not taken by this operator")
        return self._call_prefill(*args, block_mask=block_mask, cache_seqlens=cache_seqlens)
