"""Canonicaliser: traced spec -> kernel selection.

The reference prints every traced spec as kernel source
(attention_engine/core/lower/lower.py:319-559, lower_linear.py:138-409).  This
package ships a fixed kernel library instead, so a traced spec is reduced to a
small normal form and matched against the library:

* ``score_mod`` is reduced algebraically to ``act(a * score [* T] + b + t + e)``
  with ``act`` in {identity, sigmoid, relu, cap * tanh}, ``a``/``b`` python
  constants, ``t`` an optional one-element custom tensor, ``T`` an optional
  [.., seq_len, seq_len_kv] custom tensor (an element-wise score multiplier)
  and ``e`` a sum of score-free terms: custom tensors of any of the shape
  classes of core/lower/lower.py:561-615 (additive [.., seq_len, seq_len_kv]
  tiles, seq_len_kv vectors, per-row and per-head tensors) and terms linear
  in ``q_idx`` / ``kv_idx`` (ALiBi: slope[h] * (kv_idx - q_idx));
* the ``OnlineFunc`` is identified behaviourally: its traced ``online_fwd`` /
  ``online_fwd_epilogue`` are run by the spec interpreter on random tiles and
  compared with each library row function, so algebraically equivalent
  spellings of the same row function are accepted; its ``forward``,
  ``backward`` and ``combine`` are checked the same way against what the
  backward and split-KV combine kernels compute;
* the linear-attention mods are reduced to a q scale, a per-token v scale and
  a traced decay function.

Anything outside the library raises ``NotImplementedError`` naming what was not
recognised; nothing is silently approximated.
"""
from __future__ import annotations

import itertools
import math
from dataclasses import dataclass, field
from typing import Dict, Optional

import torch

from .eager import evaluate, leaves
from .transform.core import SymbolicArray, SymbolScalar, Var

SEQ_TOKENS = ("seq_len", "seq_len_kv")


# ---------------------------------------------------------------------------
# score_mod: algebraic reduction
# ---------------------------------------------------------------------------
@dataclass
class Affine:
    """a * score * [mask] + sum_t coef_t * t + c + sum_m coef_m * m   (t: one-element tensors; m: score-free
    monomials, tuples of factors "t:<custom tensor>", "i:q_idx", "i:kv_idx", sorted)"""
    a: float = 0.0
    mask: Optional[str] = None
    tensors: Dict[str, float] = field(default_factory=dict)
    c: float = 0.0
    tile: Optional[str] = None   # a bare [.., seq_len, seq_len_kv] tensor (not yet multiplied with the score, nor added to anything)
    extra: Dict[tuple, float] = field(default_factory=dict)

    def is_const(self):
        return self.a == 0.0 and not self.tensors and self.tile is None and not self.extra

    def settled(self):
        """The same value with a bare tile counted as an additive term."""
        if self.tile is None:
            return self
        extra = dict(self.extra)
        extra[("t:" + self.tile,)] = extra.get(("t:" + self.tile,), 0.0) + 1.0
        return Affine(self.a, self.mask, dict(self.tensors), self.c, None, extra)

    def scaled(self, f: float):
        x = self.settled()
        return Affine(x.a * f, x.mask, {k: v * f for k, v in x.tensors.items()}, x.c * f, None, {k: v * f for k, v in x.extra.items()})

    def score_free_poly(self):
        """{monomial: coefficient} of a term without the score (one-element tensors as factors "o:<name>")."""
        x = self.settled()
        assert x.a == 0.0
        poly = dict(x.extra)
        if x.c != 0.0:
            poly[()] = x.c
        for k, v in x.tensors.items():
            poly[("o:" + k,)] = v
        return poly

    @staticmethod
    def from_poly(poly):
        out = Affine()
        for mono, coef in poly.items():
            if coef == 0.0:
                continue
            if mono == ():
                out.c += coef
            elif len(mono) == 1 and mono[0].startswith("o:"):
                out.tensors[mono[0][2:]] = out.tensors.get(mono[0][2:], 0.0) + coef
            else:
                out.extra[mono] = out.extra.get(mono, 0.0) + coef
        return out


@dataclass
class Activated:
    """p * fn(inner) + q"""
    fn: str
    inner: Affine
    p: float = 1.0
    q: float = 0.0


@dataclass
class ScoreForm:
    activation: str            # "identity" | "sigmoid" | "relu"
    scale: float
    bias: float
    bias_tensor: Optional[str]
    mask_tensor: Optional[str]
    # score-free additive terms inside the activation: {monomial: coefficient}, see Affine
    extra: Dict[tuple, float] = field(default_factory=dict)
    # softcap: the activation's argument x is replaced by softcap * tanh(x) (identity activation only)
    softcap: Optional[float] = None


def _is_tile_tensor(sym) -> bool:
    return "seq_len_kv" in sym.shape_idx


def _reduce_score(sym: SymbolScalar, score_id: int, custom: dict):
    t = sym.code.type
    if id(sym) == score_id:
        return Affine(a=1.0)
    if t == "Const":
        return Affine(c=float(sym.code.value))
    if t == "Var" and not sym.prev:
        name = sym.varname
        if name in custom and custom[name] is sym:
            if _is_tile_tensor(sym) and "seq_len" in sym.shape_idx:
                return Affine(tile=name)
            numel_tokens = [x for x in sym.shape_idx if x not in ("1",)]
            if numel_tokens:
                for tok in numel_tokens:
                    if tok not in ("batch", "heads", "seq_len", "seq_len_kv"):
                        raise NotImplementedError(f"score_mod: custom tensor '{name}' of shape {sym.shape_idx}: literal sizes other than 1")
                return Affine(extra={("t:" + name,): 1.0})
            return Affine(tensors={name: 1.0})
        if name in ("q_idx", "kv_idx"):
            return Affine(extra={("i:" + name,): 1.0})
        try:
            return Affine(c=float(sym.code.name))
        except ValueError:
            raise NotImplementedError(f"score_mod uses '{name}', which the kernel library does not provide "
                                      f"(of the index arguments only q_idx and kv_idx are)") from None
    ins = [_reduce_score(p, score_id, custom) for p in sym.prev]
    if t == "Neg":
        return _scale(ins[0], -1.0)
    if t in ("Add", "Sub"):
        x, y = ins
        if t == "Sub":
            y = _scale(y, -1.0)
        return _add(x, y)
    if t == "Mul":
        x, y = ins
        if isinstance(y, Affine) and y.is_const():
            return _scale(x, y.c)
        if isinstance(x, Affine) and x.is_const():
            return _scale(y, x.c)
        if isinstance(x, Affine) and isinstance(y, Affine):
            for u, w in ((x, y), (y, x)):
                if (w.tile is not None and not w.extra and u.tile is None and u.mask is None and not u.tensors and u.c == 0.0
                        and not u.extra and u.a != 0.0):
                    return Affine(a=u.a, mask=w.tile)
            if x.a == 0.0 and y.a == 0.0:   # two score-free terms: multiply out
                poly = {}
                for mx, cx in x.score_free_poly().items():
                    for my, cy in y.score_free_poly().items():
                        mono = tuple(sorted(mx + my))
                        poly[mono] = poly.get(mono, 0.0) + cx * cy
                return Affine.from_poly(poly)
        raise NotImplementedError("score_mod: product of two non-constant terms other than score * tile tensor and products of "
                                  "score-free terms")
    if t == "Div":
        x, y = ins
        if isinstance(y, Affine) and y.is_const():
            return _scale(x, 1.0 / y.c)
        if isinstance(x, Affine) and x.is_const() and isinstance(y, Activated) and y.fn == "exp" and y.p == 1.0 and y.q == 1.0:
            # c / (1 + exp(u)) = c * sigmoid(-u)
            return Activated("sigmoid", y.inner.scaled(-1.0), p=x.c, q=0.0)
        raise NotImplementedError("score_mod: division by a non-constant term")
    if t in ("Tanh", "Exp"):
        (x,) = ins
        if not isinstance(x, Affine):
            raise NotImplementedError(f"score_mod: {t} of a non-affine term")
        return Activated(t.lower(), x.settled())
    if t == "Max":
        x, y = ins
        if isinstance(y, Affine) and y.is_const() and y.c == 0.0 and isinstance(x, Affine):
            return Activated("relu", x.settled())
        if isinstance(x, Affine) and x.is_const() and x.c == 0.0 and isinstance(y, Affine):
            return Activated("relu", y.settled())
        raise NotImplementedError("score_mod: max() other than max(affine, 0)")
    raise NotImplementedError(f"score_mod: op {t} is not in the kernel library")


def _scale(x, f: float):
    if isinstance(x, Affine):
        return x.scaled(f)
    return Activated(x.fn, x.inner, x.p * f, x.q * f)


def _add(x, y):
    if isinstance(x, Affine) and isinstance(y, Affine):
        x, y = x.settled(), y.settled()   # (a bare tile in a sum is an additive bias tile)
        if x.a != 0.0 and y.a != 0.0 and x.mask != y.mask:
            raise NotImplementedError("score_mod: score terms with different multipliers")
        tensors = dict(x.tensors)
        for k, v in y.tensors.items():
            tensors[k] = tensors.get(k, 0.0) + v
        extra = dict(x.extra)
        for k, v in y.extra.items():
            extra[k] = extra.get(k, 0.0) + v
        return Affine(x.a + y.a, x.mask if x.a != 0.0 else y.mask, tensors, x.c + y.c, None, {k: v for k, v in extra.items() if v != 0.0})
    if isinstance(x, Activated) and isinstance(y, Affine) and y.is_const():
        return Activated(x.fn, x.inner, x.p, x.q + y.c)
    if isinstance(y, Activated) and isinstance(x, Affine) and x.is_const():
        return Activated(y.fn, y.inner, y.p, y.q + x.c)
    raise NotImplementedError("score_mod: sum of two activated terms")


def _close(a: float, b: float) -> bool:
    return abs(a - b) <= 1e-6 * max(1.0, abs(b))


def canonicalize_score_mod(score_mod, custom_fwd_inputs) -> ScoreForm:
    score = SymbolScalar("scores", Var("scores"), shape_idx=["block_M", "block_N"])
    idx = [SymbolScalar(n, Var(n)) for n in ("b", "h", "q_idx", "kv_idx")]
    out = score_mod(score, custom_fwd_inputs, *idx) if score_mod is not None else score
    form = _reduce_score(out, id(score), custom_fwd_inputs.input_tensors)
    softcap = None
    if isinstance(form, Activated):
        inner, act = form.inner, None
        if form.fn == "tanh" and _close(form.p, 0.5) and _close(form.q, 0.5):
            inner, act = inner.scaled(2.0), "sigmoid"      # (tanh(x)+1)/2 = sigmoid(2x)
        elif form.fn == "tanh" and _close(form.q, 0.0) and form.p > 0:
            act, softcap = "identity", float(form.p)        # soft-capping: cap * tanh(x), then the row function
        elif form.fn == "sigmoid" and _close(form.p, 1.0) and _close(form.q, 0.0):
            act = "sigmoid"
        elif form.fn == "relu" and _close(form.q, 0.0) and form.p > 0:
            inner, act = inner.scaled(form.p), "relu"      # p*max(x,0) = max(p*x,0) for p>0
        if act is None:
            raise NotImplementedError(f"score_mod: {form.p}*{form.fn}(.)+{form.q} is not a library activation")
    else:
        inner, act = form.settled(), "identity"
    if inner.tile is not None or inner.a == 0.0:
        raise NotImplementedError("score_mod does not depend linearly on the score")
    for mono in inner.extra:
        n_idx = sum(f.startswith("i:") for f in mono)
        if n_idx > 1 or (n_idx == 1 and len(mono) > 2) or (n_idx == 0 and len(mono) > 1):
            raise NotImplementedError(f"score_mod: the additive term {' * '.join(f[2:] for f in mono)} is not in the kernel library "
                                      "(sums of custom tensors, and q_idx / kv_idx times a constant or a per-head tensor, are)")
        if n_idx == 1 and len(mono) == 2:
            other = [f for f in mono if not f.startswith("i:")][0]
            sym = custom_fwd_inputs.input_tensors.get(other[2:])
            toks = [x for x in (sym.shape_idx if sym is not None else []) if x != "1"]
            if toks not in ([], ["heads"]):
                raise NotImplementedError(f"score_mod: {mono}: an index may be multiplied by a constant, a one-element or a per-head tensor")
    bias_tensor = None
    if len(inner.tensors) == 1 and _close(next(iter(inner.tensors.values())), 1.0):
        (bias_tensor, _), = inner.tensors.items()          # the kernels' own bias pointer (examples/sigmoid_attn.py:17-21)
    elif inner.tensors:
        # one-element tensors with another coefficient, or several of them: additive terms like any other custom tensor
        extra = dict(inner.extra)
        for name, coef in inner.tensors.items():
            extra[("t:" + name,)] = extra.get(("t:" + name,), 0.0) + coef
        inner = Affine(inner.a, inner.mask, {}, inner.c, None, extra)
    if act != "identity" and inner.mask is not None:
        raise NotImplementedError("score_mod: activation of a tile-multiplied score")
    if inner.mask is not None and (inner.extra or softcap is not None):
        raise NotImplementedError("score_mod: additive terms / soft-capping together with a tile-multiplied score")
    return ScoreForm(act, inner.a, inner.c, bias_tensor, inner.mask, dict(inner.extra), softcap)


# ---------------------------------------------------------------------------
# OnlineFunc: behavioural identification
# ---------------------------------------------------------------------------
def _lib_softmax(s, st):
    m, r = st
    m_new = torch.maximum(m, s.amax(-1, keepdim=True))
    c = torch.exp(m - m_new)
    p = torch.exp(s - m_new)
    return p, c, (m_new, r * c + p.sum(-1, keepdim=True))


def _lib_identity(s, st):
    return s, torch.ones_like(s[..., :1]), ()


def _lib_retention(s, st):
    r_wo, r = st
    r_wo_new = r_wo + s.abs().sum(-1, keepdim=True)
    r_new = torch.clamp(r_wo_new, min=1.0)
    return s / r_new, r / r_new, (r_wo_new, r_new)


ROW_FUNCTIONS = {
    # name: (fn, state init values, epilogue(o, state) -> (o', final scale or None))
    "softmax": (_lib_softmax, (float("-inf"), 0.0), lambda o, st: (o / st[1], torch.log(st[1]) + st[0])),
    "identity": (_lib_identity, (), lambda o, st: (o, None)),
    "retention": (_lib_retention, (0.0, 0.0), lambda o, st: (o, st[1])),
}


def _random_state(name, M, gen, magnitude=1.0):
    """Plausible running statistics; ``magnitude`` scales them with the scores so
    that both sides of a clamp / max are exercised."""
    if name == "softmax":
        return (torch.randn(M, 1, generator=gen, dtype=torch.float64), torch.rand(M, 1, generator=gen, dtype=torch.float64) + 0.5)
    if name == "retention":
        r_wo = torch.rand(M, 1, generator=gen, dtype=torch.float64) * 2.0 * min(magnitude, 1.0)
        return (r_wo, torch.clamp(r_wo, min=1.0))
    return ()


def identify_online_func(online_func, return_scale: bool = False):
    """Returns the name of the library row function ``online_func`` computes; with ``return_scale`` the pair
    (name, inner scale).  The inner scale c is 1 except for a softmax that scales the scores itself,
    p = exp(c (s - m)) with lse = log r + c m (examples/mha_v2.py:44-69 spells it with exp2 and c log2 e): that is the
    library's softmax of c s, and the caller folds c into the score function.  ``None`` (examples/sigmoid_attn_v2.py:67,
    reluattn_v2.py:59) is the identity row function."""
    if online_func is None:
        return ("identity", 1.0) if return_scale else "identity"
    idx = [SymbolScalar(n, Var(n)) for n in ("b", "h", "q_idx")]
    state_syms = dict(online_func.online_rowscales)
    names = list(state_syms)
    try:
        inits = tuple(float(s.code.name) for s in state_syms.values())
    except ValueError as e:
        raise NotImplementedError(f"online_rowscales initial value not a literal: {e}") from None
    tile_in = SymbolicArray("scores_online", Var("scores_online"))
    tile_out, state_out, o_scale = online_func.online_fwd(tile_in, dict(state_syms), *idx)
    acc_in = SymbolicArray("acc_o", Var("acc_o"), shape_idx=["block_M", "dimv"])
    acc_out, finals = online_func.online_fwd_epilogue(acc_in, dict(state_syms), *idx)
    if set(state_out) != set(names):
        raise NotImplementedError("online_fwd must return every online_rowscale it was given")
    for sym in leaves([tile_out, o_scale, acc_out] + list(state_out.values()) + list(finals.values())):
        if sym.code.type == "Var" and sym is not tile_in and sym is not acc_in and all(sym is not s for s in state_syms.values()):
            try:
                float(sym.code.name)
            except ValueError:
                raise NotImplementedError(f"online_func reads '{sym.varname}', which the kernel library does not provide") from None

    gen = torch.Generator().manual_seed(1234)
    M, N, DV = 5, 7, 3
    tried = []
    for lib_name, (fn, lib_inits, epi) in ROW_FUNCTIONS.items():
        if len(lib_inits) != len(names):
            continue
        for perm in itertools.permutations(range(len(names))):
            # perm[i] = index of the user's state variable that plays library role i
            if any(not _same_init(inits[perm[i]], lib_inits[i]) for i in range(len(lib_inits))):
                continue

            def matches(c):
                # the user's running maximum is in the units of its scores, the library's in those of c * scores
                ok = True
                for magnitude in (2.0, 0.02, 0.2):
                    s = torch.randn(M, N, generator=gen, dtype=torch.float64) * magnitude
                    st = _random_state(lib_name, M, gen, magnitude)
                    env = {id(tile_in): s}
                    for i, j in enumerate(perm):
                        env[id(state_syms[names[j]])] = st[i]
                    got = evaluate([tile_out, o_scale] + [state_out[names[j]] for j in perm], env, s)
                    lib_st = (st[0] * c,) + tuple(st[1:]) if c != 1.0 else st
                    exp_p, exp_c, exp_st = fn(s * c, lib_st)
                    if c != 1.0:
                        got[2] = got[2] * c
                    ok &= _allclose(got[0], exp_p) and _allclose(got[1], exp_c)
                    ok &= all(_allclose(g, e) for g, e in zip(got[2:], exp_st))
                    o = torch.randn(M, DV, generator=gen, dtype=torch.float64)
                    env = {id(acc_in): o}
                    for i, j in enumerate(perm):
                        env[id(state_syms[names[j]])] = st[i]
                    got = evaluate([acc_out] + list(finals.values()), env, o)
                    exp_o, exp_final = epi(o, lib_st)
                    ok &= _allclose(got[0], exp_o)
                    if exp_final is None:
                        ok &= len(got) == 1
                    else:
                        ok &= len(got) == 2 and _allclose(got[1], exp_final)
                    if not ok:
                        break
                return ok

            inner = 1.0
            ok = matches(1.0)
            if not ok and lib_name == "softmax":
                # a softmax of c * scores: read c off one probability, exp(c (0 - 1)) from an empty state, then compare as above
                s = torch.tensor([[0.0, 1.0]], dtype=torch.float64)
                env = {id(tile_in): s}
                for i, j in enumerate(perm):
                    env[id(state_syms[names[j]])] = torch.full((1, 1), lib_inits[i], dtype=torch.float64)
                p0 = float(evaluate([tile_out], env, s)[0][0, 0])
                if 0.0 < p0 < 1.0:
                    inner = -math.log(p0)
                    ok = matches(inner)
            if ok:
                _check_recompute_and_combine(online_func, lib_name, inner)
                if inner != 1.0 and not return_scale:
                    raise NotImplementedError("this OnlineFunc scales the scores itself; ask for the scale with return_scale=True")
                return (lib_name, inner) if return_scale else lib_name
        tried.append(lib_name)
    raise NotImplementedError(
        f"OnlineFunc with row scales {names} (initial values {inits}) matches no library row function "
        f"(softmax, identity, retention); compared against: {tried or 'none with that many row scales'}")


def _check_recompute_and_combine(online_func, lib_name: str, inner: float = 1.0):
    """The other three methods of the contract, where the spec overrides them: ``forward`` (the probabilities again, from
    the scores and the final row scale), ``backward`` (dscores from dp: both generated into the backward kernel by
    core/lower/lower.py:425-438) and ``combine`` (the weight of every kv split, generated into the split-KV merge by
    core/lower/lower_decode.py:287-313).  The library's backward and combine kernels hold ONE version of each per row
    function; a spec whose traced version computes something else is refused instead of being silently replaced:
        softmax    forward exp(s - lse)   backward (dp - doosum) * p   combine exp(lse_i - logsumexp_i(lse))  (or the same
                   in base 2, as examples/mha_decode.py:72-80 spells it for its log2-domain lse); with an inner scale c:
                   forward exp(c s - lse), backward (dp - doosum) * p with or without the factor c (examples/mha_v2.py:79-83
                   leaves it to its template; the kernels compute the gradient of the forward either way)
        identity   forward s              backward dp
        retention  forward s / r          backward dp / r"""
    from attn_engine import OnlineFunc          # (the base class: methods left at its defaults are not looked at)
    from .transform.core import SymbolicColReduceArray
    cls = type(online_func)
    finals = list(online_func.final_rowscales)
    if lib_name != "identity" and len(finals) != 1:
        return
    gen = torch.Generator().manual_seed(4321)
    M, N, NS = 5, 7, 4
    idx = [SymbolScalar(n, Var(n)) for n in ("b", "h", "q_idx", "kv_idx")]

    def run(method, what, build):
        try:
            out_sym, env, like, expect = build()
            got = evaluate([out_sym], env, like)[0]
        except NotImplementedError:
            raise
        except Exception as e:
            raise NotImplementedError(f"OnlineFunc.{method} could not be traced: {e!r}") from None
        if not any(_allclose(got, e) for e in expect):
            raise NotImplementedError(f"OnlineFunc.{method} computes something else than the library's {what} for the {lib_name} row "
                                      "function; the kernel library holds one version of it and does not generate another")

    fin = torch.randn(M, 1, generator=gen, dtype=torch.float64)
    if lib_name == "retention":
        fin = fin.abs() + 1.0
    sc = torch.randn(M, N, generator=gen, dtype=torch.float64)
    prob = {"softmax": lambda: torch.exp(sc * inner - fin), "identity": lambda: sc, "retention": lambda: sc / fin}[lib_name]()

    if getattr(cls, "forward", None) is not OnlineFunc.forward:
        def build():
            tile = SymbolicArray("scores_fwd", Var("scores_fwd"))
            fsyms = {n: SymbolScalar(n, Var(n)) for n in finals}
            out = online_func.forward(tile, fsyms, *idx)
            env = {id(tile): sc, **{id(v): fin for v in fsyms.values()}}
            return out, env, sc, [prob]
        run("forward", "recomputation of the probabilities", build)

    if getattr(cls, "backward", None) is not OnlineFunc.backward:
        dp = torch.randn(M, N, generator=gen, dtype=torch.float64)
        doosum = torch.randn(M, 1, generator=gen, dtype=torch.float64)
        expect = {"softmax": (dp - doosum) * prob, "identity": dp, "retention": dp / fin}[lib_name]

        def build():
            dps, ps = SymbolicArray("dp", Var("dp")), SymbolicArray("p", Var("p"))
            ds = SymbolScalar("doosum", Var("doosum"))
            fsyms = {n: SymbolScalar(n, Var(n)) for n in finals}
            try:     # the signature lower.py:437-438 calls; the base class declares it without the row sums
                out = online_func.backward(dps, ps, fsyms, ds, *idx)
            except TypeError:
                out = online_func.backward(dps, ps, fsyms, *idx)
            env = {id(dps): dp, id(ps): prob, id(ds): doosum, **{id(v): fin for v in fsyms.values()}}
            return out, env, dp, [expect] if inner == 1.0 else [expect, expect * inner]
        run("backward", "score gradient", build)

    if getattr(cls, "combine", None) is not OnlineFunc.combine:
        if lib_name != "softmax":
            raise NotImplementedError("split-KV combine is only in the softmax operators of the kernel library")
        lse = torch.randn(NS, M, generator=gen, dtype=torch.float64) * 3

        def build():
            fsyms = {finals[0]: SymbolicColReduceArray(finals[0], Var(finals[0]), shape_idx=["num_split", "block_M"])}
            out = online_func.combine(fsyms)
            return out, {id(fsyms[finals[0]]): lse}, lse, [torch.softmax(lse, dim=0), torch.softmax(lse * math.log(2.0), dim=0)]
        run("combine", "log-sum-exp merge of the kv splits", build)


def _same_init(a: float, b: float) -> bool:
    return (math.isinf(a) and math.isinf(b) and a == b) or a == b


def _allclose(a, b) -> bool:
    if a.shape != b.shape:
        try:
            a, b = torch.broadcast_tensors(a, b)
        except RuntimeError:
            return False
    return bool(torch.allclose(a, b, rtol=1e-9, atol=1e-11, equal_nan=False))


# ---------------------------------------------------------------------------
# mask_mod
# ---------------------------------------------------------------------------
class _IndexNotToBeRead:
    """Stands in for the batch / head index of a mask_mod: any use of it raises."""

    def _used(self, *a, **k):
        raise _IndexWasRead()

    __eq__ = __ne__ = __lt__ = __le__ = __gt__ = __ge__ = __add__ = __radd__ = __sub__ = __rsub__ = __mul__ = __rmul__ = _used
    __truediv__ = __rtruediv__ = __floordiv__ = __rfloordiv__ = __mod__ = __rmod__ = __and__ = __rand__ = __or__ = __ror__ = _used
    __xor__ = __rxor__ = __neg__ = __invert__ = __index__ = __int__ = __float__ = __bool__ = __getitem__ = __hash__ = _used
    __torch_function__ = classmethod(lambda cls, *a, **k: (_ for _ in ()).throw(_IndexWasRead()))


class _IndexWasRead(Exception):
    pass


# a mask_mod that reads its batch / head index is compared over every (batch, head) pair (stopping at the first pair that
# differs) when the whole mask has at most this many elements -- about a second of construction time; beyond that it is
# taken to depend on them
_MASK_COMPARE_LIMIT = 1 << 28


def classify_mask(mask_mod, B, H, Sq, Skv, block_M=128, block_N=128) -> str:
    """"none" | "causal" | "other" | "other_bh".  Evaluates ``mask_mod`` densely on index grids on
    the CPU (as the reference does, over all of B and H, at block granularity: lower.py:723-740) and
    compares with the exact causal pattern.  "other": some other pattern, the same for every (batch,
    head); "other_bh": it depends on batch or head.  Both run through an element-wise keep mask built by
    the caller (the reference generates the mask_mod's code into its block-sparse kernel instead,
    blockattn_tl.py:176-190).

    Whether the pattern depends on (batch, head) is decided, not sampled: a mask_mod that never touches
    its b and h arguments (found by calling it with stand-ins that raise on any use) is evaluated once;
    one that does is evaluated for every pair and compared with the first, and where that would be more
    than 2^28 elements it counts as depending on them (always correct, possibly a larger keep mask than
    needed)."""
    if mask_mod is None:
        return "none"
    qi = torch.arange(Sq).view(Sq, 1)
    kj = torch.arange(Skv).view(1, Skv)

    def dense(b, h):
        m = mask_mod(b, h, qi, kj)
        m = m if torch.is_tensor(m) else torch.full((Sq, Skv), bool(m))
        return m.to(torch.bool).expand(Sq, Skv)

    try:
        first = dense(_IndexNotToBeRead(), _IndexNotToBeRead())
        reads_bh = False
    except (_IndexWasRead, TypeError, RuntimeError):   # the stand-in was used, or handed to something that refuses it;
        first = dense(torch.tensor(0), torch.tensor(0))  # any other error is the mask_mod's own and is raised here, the first time
        reads_bh = True
    if reads_bh and B * H > 1:
        if B * H * Sq * Skv > _MASK_COMPARE_LIMIT:
            return "other_bh"
        for b in range(B):
            for h in range(H):
                if (b or h) and not torch.equal(dense(torch.tensor(b), torch.tensor(h)), first):
                    return "other_bh"
    if Sq == Skv and torch.equal(first, qi >= kj):
        return "causal"
    if bool(first.all()):
        return "none"
    return "other"


# ---------------------------------------------------------------------------
# linear-attention mods
# ---------------------------------------------------------------------------
@dataclass
class LinearPlan:
    q_scale: float = 1.0
    v_scale_tensor: Optional[str] = None      # custom tensor ("batch","heads","seq_len") multiplying v per token
    decay_sym: Optional[SymbolScalar] = None  # traced decay_mod output (None: decay is already the log decay)
    decay_in: Optional[SymbolScalar] = None
    decay_kind: str = "identity"              # "identity" | "log" | "mul_head" | "traced"
    decay_head_tensor: Optional[str] = None


def _reduce_linear(sym, x_id, custom):
    """-> (coef, token_scale_tensor|None) with out = coef * x [* tensor]"""
    t = sym.code.type
    if id(sym) == x_id:
        return (1.0, None)
    if t == "Const":
        return ("const", float(sym.code.value))
    if t == "Var" and not sym.prev:
        if sym.varname in custom and custom[sym.varname] is sym:
            return ("tensor", sym.varname)
        raise NotImplementedError(f"mod uses unknown symbol '{sym.varname}'")
    ins = [_reduce_linear(p, x_id, custom) for p in sym.prev]
    if t in ("Mul", "Div"):
        a, b = ins
        if t == "Div":
            if b[0] != "const":
                raise NotImplementedError("mod: division by a non-constant")
            b = ("const", 1.0 / b[1])
        for u, w in ((a, b), (b, a)):
            if isinstance(u[0], float):
                if w[0] == "const":
                    return (u[0] * w[1], u[1])
                if w[0] == "tensor" and u[1] is None:
                    return (u[0], w[1])
        if a[0] == "const" and b[0] == "const":
            return ("const", a[1] * b[1])
    if t == "Neg" and isinstance(ins[0][0], float):
        return (-ins[0][0], ins[0][1])
    raise NotImplementedError(f"mod: op {t} is not a scaling of its input")


def canonicalize_linear_mods(q_mod, k_mod, v_mod, decay_mod, custom_io) -> LinearPlan:
    custom = custom_io.input_tensors if custom_io is not None else {}
    plan = LinearPlan()

    def trace(mod, name, shape):
        x = SymbolScalar(name, Var(name), shape_idx=shape)
        return x, mod(x, custom_io)

    for mod, name in ((q_mod, "q"), (k_mod, "k")):
        if mod is None:
            continue
        x, out = trace(mod, name, ["batch", "heads", "seq_len", "dim"])
        coef, tensor = _reduce_linear(out, id(x), custom)
        if tensor is not None:
            raise NotImplementedError(f"{name}_mod: multiplying by a tensor is not in the kernel library")
        plan.q_scale *= coef       # the operator is bilinear in q and k: a k scale folds into the q scale
    if v_mod is not None:
        x, out = trace(v_mod, "v", ["batch", "heads", "seq_len", "dimv"])
        coef, tensor = _reduce_linear(out, id(x), custom)
        plan.q_scale *= coef
        if tensor is not None:
            shp = custom[tensor].shape_idx
            if shp != ["batch", "heads", "seq_len"]:
                raise NotImplementedError(f"v_mod: tensor '{tensor}' must have shape (batch, heads, seq_len), got {shp}")
            plan.v_scale_tensor = tensor
    if decay_mod is not None:
        x, out = trace(decay_mod, "decay", ["batch", "heads", "seq_len"])
        plan.decay_sym, plan.decay_in = out, x
        plan.decay_kind = "traced"
        if out.code.type == "Log" and out.prev[0] is x:
            plan.decay_kind = "log"
        elif out.code.type == "Mul":
            a, b = out.prev
            other = b if a is x else a if b is x else None
            if other is not None and other.code.type == "Var" and other.varname in custom \
                    and custom[other.varname].shape_idx == ["1", "heads"]:
                plan.decay_kind, plan.decay_head_tensor = "mul_head", other.varname
    return plan
