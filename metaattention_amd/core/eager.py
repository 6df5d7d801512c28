"""Interpreter for traced specs on torch tensors.

Gives a traced ``SymbolScalar`` graph its meaning by evaluating it with
PyTorch ops.  Op semantics are the mathematical ones of the reference's
PyTorch printer (attention_engine/core/codegen/tl_gen.py:236-303): Exp is
e^x, Log is ln x, row reductions run over the last (kv) axis.  Used by the
canonicaliser to identify which library row function a user's ``OnlineFunc``
computes, and by host-side tests that validate tracing against the oracle.  It
is not an execution backend of the operators: those only run the HIP kernels.
"""
from __future__ import annotations

from typing import Dict, Iterable

import torch

from .transform.core import SymbolScalar

_UNARY = {
    "Neg": torch.neg, "Abs": torch.abs, "Exp": torch.exp, "Exp2": torch.exp2,
    "Log": torch.log, "Log2": torch.log2, "Tanh": torch.tanh,
}
_BINARY = {
    "Add": torch.add, "Sub": torch.sub, "Mul": torch.mul, "Div": torch.div, "Max": torch.maximum,
}


def _const_of(name: str) -> float:
    """Leaf ``Var`` names that are literals: "-inf", "0.0", "1", ..."""
    return float(name)


def evaluate(outputs: Iterable[SymbolScalar], env: Dict[int, torch.Tensor], like: torch.Tensor):
    """Evaluates traced values.  ``env`` maps ``id(symbol)`` of the trace's
    input symbols to tensors; row statistics are kept with a trailing unit
    axis so they broadcast against tiles.  ``like`` supplies dtype/device for
    constants."""
    cache: Dict[int, torch.Tensor] = dict(env)

    def const(v):
        return torch.tensor(float(v), dtype=like.dtype, device=like.device)

    def ev(s: SymbolScalar):
        key = id(s)
        if key in cache:
            return cache[key]
        t = s.code.type
        if t == "Const":
            out = const(s.code.value)
        elif t == "Var":
            try:
                out = const(_const_of(s.code.name))
            except ValueError:
                raise KeyError(f"unbound symbol '{s.varname}' (Var {s.code.name!r}) in traced spec") from None
        elif t in _UNARY:
            out = _UNARY[t](ev(s.prev[0]))
        elif t in _BINARY:
            a, b = ev(s.prev[0]), ev(s.prev[1])
            out = _BINARY[t](a, b)
        elif t == "ReduceSum":
            out = ev(s.prev[0]).sum(dim=-1, keepdim=True)
        elif t == "ReduceMax":
            out = ev(s.prev[0]).amax(dim=-1, keepdim=True)
        elif t == "ReduceAbsSum":
            out = ev(s.prev[0]).abs().sum(dim=-1, keepdim=True)
        elif t == "ColReduceSum":
            out = ev(s.prev[0]).sum(dim=0, keepdim=True)
        elif t == "ColReduceMax":
            out = ev(s.prev[0]).amax(dim=0, keepdim=True)
        elif t == "ColReduceAbsSum":
            out = ev(s.prev[0]).abs().sum(dim=0, keepdim=True)
        else:
            raise NotImplementedError(f"op {t} has no forward meaning")
        cache[key] = out
        return out

    return [ev(o) for o in outputs]


def leaves(outputs: Iterable[SymbolScalar]):
    """All input symbols (no producers) reachable from ``outputs``."""
    seen, out = set(), []

    def walk(s):
        if id(s) in seen:
            return
        seen.add(id(s))
        if not s.prev:
            out.append(s)
        for p in s.prev:
            walk(p)

    for o in outputs:
        walk(o)
    return out


_AXIS = {"batch": 0, "heads": 1, "seq_len": 2, "seq_len_kv": 3}


def custom_tensor_view(t: torch.Tensor, shape_tokens) -> torch.Tensor:
    """Reshapes a custom input to a [B|1, H|1, Sq|1, Skv|1] broadcastable view
    according to its symbolic shape (dimension tokens map to axes the way
    core/lower/lower.py:32-39 maps them to block indices; literal sizes keep
    their position when the tensor is 4-D and are unit axes otherwise)."""
    toks = [str(x) for x in shape_tokens]
    if len(toks) == 4:
        return t
    shape = [1, 1, 1, 1]
    for tok, size in zip(toks, t.shape):
        if tok in _AXIS:
            shape[_AXIS[tok]] = size
        elif size != 1:
            raise ValueError(f"cannot place literal dimension {tok} of a {len(toks)}-D custom tensor")
    return t.reshape(shape)


def attention_by_spec(q, k, v, custom_tensors, *, score_mod, mask_mod, online_func, custom_fwd_inputs,
                      mask_value="-inf", block_n: int = 0):
    """Runs a parallel-attention spec literally, the way the reference kernel
    does (attn_tl.py:123-188): for each kv block, scores = q.k^T with the mask
    pre-loaded as 0 / -inf, ``score_mod``, ``online_fwd``, rescale the
    accumulator by ``o_scale``, accumulate P.V; then ``online_fwd_epilogue``.
    q,k,v are BSHD; returns (o [B,Sq,H,Dv], final_rowscales dict of [B,H,Sq]).
    ``block_n=0`` processes each row in one block."""
    from .transform.core import SymbolicArray, SymbolScalar as SS, Var
    B, Sq, H, _ = q.shape
    Skv = k.shape[1]
    bn = Skv if block_n <= 0 else block_n
    qf, kf, vf = (x.permute(0, 2, 1, 3).to(torch.float32) for x in (q, k, v))   # BHSD
    names = list(custom_fwd_inputs.input_tensors)
    assert len(custom_tensors) == len(names), "custom tensors must follow CustomIO order"
    views = {n: custom_tensor_view(t.to(torch.float32), custom_fwd_inputs.input_tensors[n].shape_idx)
             for n, t in zip(names, custom_tensors)}
    idx_b, idx_h, idx_q, idx_k = (SS(n, Var(n)) for n in ("b", "h", "q_idx", "kv_idx"))

    # trace once
    score_in = SS("scores", Var("scores"), shape_idx=["block_M", "block_N"])
    score_out = score_mod(score_in, custom_fwd_inputs, idx_b, idx_h, idx_q, idx_k)
    tile_in = SymbolicArray("scores_online", Var("scores_online"))
    state_in = dict(online_func.online_rowscales)
    tile_out, state_out, o_scale = online_func.online_fwd(tile_in, dict(state_in), idx_b, idx_h, idx_q)
    acc_in = SymbolicArray("acc_o", Var("acc_o"), shape_idx=["block_M", "dimv"])
    acc_out, finals = online_func.online_fwd_epilogue(acc_in, dict(state_in), idx_b, idx_h, idx_q)

    state = {n: torch.full((B, H, Sq, 1), _const_of(s.code.name), dtype=torch.float32, device=q.device)
             for n, s in state_in.items()}
    acc = torch.zeros(B, H, Sq, v.shape[-1], dtype=torch.float32, device=q.device)
    qi = torch.arange(Sq, device=q.device).view(1, 1, Sq, 1)
    for n0 in range(0, Skv, bn):
        n1 = min(n0 + bn, Skv)
        s = qf @ kf[:, :, n0:n1].transpose(-1, -2)
        if mask_mod is not None and mask_value == "-inf":
            kj = torch.arange(n0, n1, device=q.device).view(1, 1, 1, -1)
            keep = mask_mod(torch.arange(B, device=q.device).view(B, 1, 1, 1),
                            torch.arange(H, device=q.device).view(1, H, 1, 1), qi, kj)
            s = s + torch.where(keep, 0.0, float("-inf"))
        env = {id(score_in): s}
        for n, sym in custom_fwd_inputs.input_tensors.items():
            vw = views[n]
            env[id(sym)] = vw[..., n0:n1] if vw.shape[-1] == Skv and Skv > 1 else vw
        (s,) = evaluate([score_out], env, s)
        env = {id(tile_in): s, **{id(state_in[n]): state[n] for n in state_in}}
        res = evaluate([tile_out, o_scale] + [state_out[n] for n in state_in], env, s)
        p, osc = res[0], res[1]
        state = {n: r.expand(B, H, Sq, 1) for n, r in zip(state_in, res[2:])}
        acc = acc * osc + p.to(q.dtype).to(torch.float32) @ vf[:, :, n0:n1]
    env = {id(acc_in): acc, **{id(state_in[n]): state[n] for n in state_in}}
    res = evaluate([acc_out] + list(finals.values()), env, acc)
    out = res[0].permute(0, 2, 1, 3)
    return out, {n: r.expand(B, H, Sq, 1).squeeze(-1) for n, r in zip(finals, res[1:])}
