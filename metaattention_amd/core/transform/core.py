"""Symbolic values user specs are written against, and block-mask helpers.

API surface of attention_engine/core/transform/core.py:36-349 and :352-506:
``SymbolScalar`` (operator overloads + named methods build a trace),
``SymbolicArray.get_reduce`` (row reductions), ``SymbolicColReduceArray``
(column reductions, used by split-KV ``combine``), ``SymbolicTensor`` /
``SymbolicConst`` / ``CustomIO`` (custom inputs), and ``create_mask`` /
``create_block_mask`` / ``is_causal_mask`` / ``is_less_causal_mask``.

A trace is the graph of ``SymbolScalar`` objects linked through ``prev``; each
carries the op tag in ``code.type``.  Nothing here emits source text: the
trace is consumed by the canonicaliser, which selects a pre-built kernel, and
by the spec interpreter.  The backward kernels of the library hold each
family's derivative themselves, so the reverse-mode pass the reference runs
over the trace (:119-199) is not needed to build them.
"""
from __future__ import annotations

from typing import Literal, Optional

import torch

from . import graph as G
from .graph import Var, Const  # noqa: F401  (re-exported: users import Var from here)


class SymbolScalar:
    """A traced value.  ``shape_idx`` names its dimensions symbolically
    (e.g. ``["block_M", "block_N"]`` for a score tile, ``["block_M"]`` for a
    row statistic)."""

    def __init__(self, varname: str, value: G.Node, prev=(), shape_idx=("block_M",),
                 require_grad: bool = True, dtype: str = "float"):
        self.varname = varname
        self.code = value
        self.prev = list(prev)
        self.shape_idx = [str(i) for i in shape_idx]
        self.require_grad = require_grad
        self.dtype = dtype
        self.count = 0          # number of consumers (kept for API compatibility)
        self.use_list = []
        self.allow_reuse = True
        self.grad = None

    # -- bookkeeping kept so specs written for the reference keep working
    def set_allow_reuse(self, allow_reuse: bool):
        self.allow_reuse = allow_reuse

    def clear_usecount(self):
        self.count = 0
        self.use_list.clear()

    def clear_visit(self):
        pass

    def clear_codegen(self):
        self.clear_usecount()

    @property
    def name(self):
        return self.varname

    @property
    def shape(self):
        return list(self.shape_idx)

    def __repr__(self):
        return f"SymbolScalar({self.varname}: {self.code.type}, shape={self.shape_idx})"

    # -- tracing
    def op(self, code, others=(), shape_idx=None, varname_suffix: Optional[str] = None):
        """Applies node class ``code`` to ``self`` and ``others`` (python numbers
        become constants) and returns the traced result."""
        operands = []
        for other in others:
            if isinstance(other, (int, float)):
                other = SymbolicConst(other)
            elif not isinstance(other, SymbolScalar):
                raise TypeError(f"cannot trace operand of type {type(other).__name__}")
            operands.append(other)
        if shape_idx is None:
            # result takes the widest operand shape (row statistic op tile -> tile)
            shape_idx = max([self.shape_idx] + [o.shape_idx for o in operands], key=len)
        name = self.varname if varname_suffix is None else f"{self.varname}_{varname_suffix}"
        node = code(*[x.code for x in [self] + operands])
        out = SymbolScalar(f"{name}_{self.count}", node, [self] + operands, shape_idx)
        if isinstance(self, (SymbolicArray, SymbolicColReduceArray)) and len(shape_idx) == len(self.shape_idx):
            out.__class__ = self.__class__
        for x in [self] + operands:
            x.use_list.append(out)
            x.count += 1
        return out

    def _rop(self, code, other):
        return SymbolicConst(other).op(code, [self], shape_idx=self.shape_idx)

    def __add__(self, other): return self.op(G.Add, [other])
    def __radd__(self, other): return self.op(G.Add, [other])
    def __sub__(self, other): return self.op(G.Sub, [other])
    def __rsub__(self, other): return self._rop(G.Sub, other)
    def __mul__(self, other): return self.op(G.Mul, [other])
    def __rmul__(self, other): return self.op(G.Mul, [other])
    def __truediv__(self, other): return self.op(G.Div, [other])
    def __rtruediv__(self, other): return self._rop(G.Div, other)
    def __neg__(self): return self.op(G.Neg)
    def abs(self): return self.op(G.Abs)
    def tanh(self): return self.op(G.Tanh)
    def exp(self): return self.op(G.Exp)
    def exp2(self): return self.op(G.Exp2)
    def log(self): return self.op(G.Log)
    def log2(self): return self.op(G.Log2)
    def max(self, other): return self.op(G.Max, [other])
    def maxbwd(self, a, b): return self.op(G.MaxBwd, [a, b])

    def backward(self, grad=None):
        raise NotImplementedError("a traced score is not differentiated symbolically here: the gradients of the canonical score "
                                  "forms come from the library's backward kernels, through the engine's autograd function")


class SymbolicArray(SymbolScalar):
    """2-D tile handed to ``OnlineFunc.online_fwd``; ``get_reduce`` reduces
    over the last (kv) dimension."""

    def __init__(self, varname: str = "", code: G.Node = None, prev=(), shape_idx=("block_M", "block_N")):
        super().__init__(varname, code if code is not None else Var(" "), prev, shape_idx)

    _ROW = {"sum": G.ReduceSum, "max": G.ReduceMax, "abssum": G.ReduceAbsSum}

    def get_reduce(self, op: Literal["sum", "max", "abssum"]):
        if op not in self._ROW:
            raise NotImplementedError(op)
        return self.op(self._ROW[op], shape_idx=self.shape_idx[:-1], varname_suffix=op)


class SymbolicColReduceArray(SymbolScalar):
    """[num_split, rows] array handed to ``OnlineFunc.combine``; ``get_reduce``
    reduces over the first (split) dimension."""

    def __init__(self, varname: str = "", code: G.Node = None, prev=(), shape_idx=("block_M", "block_N")):
        super().__init__(varname, code if code is not None else Var(" "), prev, shape_idx)

    _COL = {"sum": G.ColReduceSum, "max": G.ColReduceMax, "abssum": G.ColReduceAbsSum}

    def get_reduce(self, op: Literal["sum", "max", "abssum"]):
        if op not in self._COL:
            raise NotImplementedError(op)
        return self.op(self._COL[op], shape_idx=self.shape_idx[:-2] + [self.shape_idx[-1]], varname_suffix=op)


class SymbolicTensor(SymbolScalar):
    """A custom input tensor; ``shape`` entries are ints or the tokens
    "batch", "heads", "seq_len", "seq_len_kv"."""

    def __init__(self, varname: str, shape: tuple):
        super().__init__(varname, Var(varname), shape_idx=[str(i) for i in shape])


class SymbolicConst(SymbolScalar):
    def __init__(self, value):
        super().__init__(f"float({value})", Const(value), prev=[], shape_idx=[], require_grad=False)


class CustomIO:
    """Ordered name -> symbolic tensor map.  The operator takes the real
    tensors positionally, after q, k, v, in this dict's order."""

    def __init__(self, input_tensors: Optional[dict] = None):
        self.input_tensors = {k: SymbolicTensor(k, v) for k, v in (input_tensors or {}).items()}


# ---------------------------------------------------------------------------
# mask helpers
# ---------------------------------------------------------------------------
def create_mask(mod_fn, B: Optional[int], H: Optional[int], Q_LEN: int, KV_LEN: int, device: str = "cuda") -> torch.Tensor:
    """Dense [B,H,Q_LEN,KV_LEN] boolean evaluation of ``mod_fn(b,h,q_idx,kv_idx)``
    (same contract as core.py:352-398, which maps the function over index
    vectors; here the function is simply applied to broadcast index grids)."""
    B, H = B or 1, H or 1
    b = torch.arange(B, device=device).view(B, 1, 1, 1)
    h = torch.arange(H, device=device).view(1, H, 1, 1)
    m = torch.arange(Q_LEN, device=device).view(1, 1, Q_LEN, 1)
    n = torch.arange(KV_LEN, device=device).view(1, 1, 1, KV_LEN)
    mask = mod_fn(b, h, m, n)
    if not torch.is_tensor(mask):
        mask = torch.full((1, 1, 1, 1), bool(mask), device=device)
    return mask.to(torch.bool).expand(B, H, Q_LEN, KV_LEN)


def _convert_mask_to_block_mask(mask: torch.Tensor, Q_BLOCK_SIZE=128, KV_BLOCK_SIZE=128, separate_full_blocks=False):
    """Pools a dense mask to blocks: int8 [B,H,ceil(Q/bq),ceil(KV/bk)], 1 where
    the block holds any kept element (or, with ``separate_full_blocks``, the
    pair (partial, full))."""
    assert mask.dtype == torch.bool
    while mask.dim() < 4:
        mask = mask.unsqueeze(0)
    B, H, Q, KV = mask.shape
    nq, nk = -(-Q // Q_BLOCK_SIZE), -(-KV // KV_BLOCK_SIZE)
    padded = torch.zeros(B, H, nq * Q_BLOCK_SIZE, nk * KV_BLOCK_SIZE, dtype=torch.bool, device=mask.device)
    padded[:, :, :Q, :KV] = mask
    counts = padded.view(B, H, nq, Q_BLOCK_SIZE, nk, KV_BLOCK_SIZE).sum(dim=(3, 5))
    if separate_full_blocks:
        full = counts == Q_BLOCK_SIZE * KV_BLOCK_SIZE
        return ((counts > 0) & ~full).to(torch.int8), full.to(torch.int8)
    return (counts > 0).to(torch.int8), None


def create_block_mask(mask_mod, B, H, QLen, KVLen, device, Q_BLOCK_SIZE=None, KV_BLOCK_SIZE=None):
    """Block-level mask of ``mask_mod`` (core.py:492-506)."""
    dense = create_mask(mask_mod, B, H, QLen, KVLen, device)
    return _convert_mask_to_block_mask(dense, Q_BLOCK_SIZE or 128, KV_BLOCK_SIZE or 128)[0]


def is_causal_mask(mask_tensor, block_M, block_N) -> torch.Tensor:
    """True when the block mask equals the block pattern of an exact causal mask:
    block (i, j) is kept iff its first kv index is below the block's last q
    index + 1 (core.py:455-470)."""
    _, _, M, N = mask_tensor.shape
    qi = torch.arange(M, device=mask_tensor.device).view(M, 1)
    kj = torch.arange(N, device=mask_tensor.device).view(1, N)
    return torch.all(mask_tensor.bool() == ((qi + 1) * block_M > kj * block_N))


def is_less_causal_mask(mask_tensor, block_M, block_N) -> torch.Tensor:
    """True when every block lying entirely above the diagonal is empty, so a
    causal loop bound skips nothing that is kept (core.py:472-488)."""
    _, _, M, N = mask_tensor.shape
    qi = torch.arange(M, device=mask_tensor.device).view(M, 1)
    kj = torch.arange(N, device=mask_tensor.device).view(1, N)
    above = (qi + 1) * block_M - 1 < kj * block_N
    return torch.all(mask_tensor[..., above] == 0)


def create_block_idx(mask_mod, B, H, QLen, KVLen, device, Q_BLOCK_SIZE=None, KV_BLOCK_SIZE=None):
    return torch.nonzero(create_block_mask(mask_mod, B, H, QLen, KVLen, device, Q_BLOCK_SIZE, KV_BLOCK_SIZE), as_tuple=False)
