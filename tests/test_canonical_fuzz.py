"""Random score_mod expressions against the canonicaliser (no GPU).  An expression is generated twice over, once on the
tracer's symbols and once on plain numbers: an affine function of the score, wrapped in nested scalings, divisions and
sums with score-free terms (custom tensors of every class, constants, q_idx / kv_idx times constants or a per-head
tensor), optionally inside one of the library's activations or a soft cap.  Whatever form the canonicaliser returns must
take the expression's own value at random points; a refusal is allowed only where the message names a limit of the kernel
library (none is hit by this generator)."""
import math
import random

import pytest

from core import CustomIO
from core.canonical import canonicalize_score_mod

IO = CustomIO({"rel": (1, "heads", "seq_len", "seq_len_kv"), "colv": ("seq_len_kv",), "rowt": ("batch", "heads", "seq_len"),
               "slopes": ("heads",), "b1": (1,)})
T = IO.input_tensors
VALUE = {"rel": 0.37, "colv": -1.3, "rowt": 0.81, "slopes": 0.05, "b1": -0.6}      # a number per custom tensor


def _score_free(rng, depth):
    """(symbolic builder, numeric builder) of a term without the score"""
    kinds = ["const", "tensor", "index", "index_slope", "sum", "scaled", "neg", "index_difference"] if depth > 0 else ["const", "tensor", "index"]
    kind = rng.choice(kinds)
    if kind == "const":
        c = round(rng.uniform(-2, 2), 3)
        return (lambda e: c), (lambda e: c)
    if kind == "tensor":
        name = rng.choice(["rel", "colv", "rowt", "b1"])
        return (lambda e: T[name]), (lambda e: VALUE[name])
    if kind == "index":
        which, c = rng.choice(["q", "k"]), round(rng.uniform(-0.1, 0.1), 4)
        return (lambda e: e[which] * c), (lambda e: e[which] * c)
    if kind == "index_slope":
        which = rng.choice(["q", "k"])
        return (lambda e: T["slopes"] * e[which]), (lambda e: VALUE["slopes"] * e[which])
    if kind == "index_difference":
        c = round(rng.uniform(-0.1, 0.1), 4)
        return (lambda e: (e["q"] - e["k"]) * c), (lambda e: (e["q"] - e["k"]) * c)
    a, an = _score_free(rng, depth - 1)
    if kind == "neg":
        return (lambda e: -a(e)), (lambda e: -an(e))
    if kind == "scaled":
        c = round(rng.uniform(-2, 2), 3)
        return ((lambda e: a(e) * c), (lambda e: an(e) * c)) if rng.random() < 0.5 else ((lambda e: c * a(e)), (lambda e: c * an(e)))
    b, bn = _score_free(rng, depth - 1)
    return ((lambda e: a(e) + b(e)), (lambda e: an(e) + bn(e))) if rng.random() < 0.5 else ((lambda e: a(e) - b(e)), (lambda e: an(e) - bn(e)))


def _affine(rng, depth):
    """(symbolic builder, numeric builder) of a function that is affine in the score e["s"]"""
    if depth == 0:
        return (lambda e: e["s"]), (lambda e: e["s"])
    a, an = _affine(rng, depth - 1)
    kind = rng.choice(["scale", "div", "add", "radd", "sub", "nest"])
    if kind == "scale":
        c = round(rng.uniform(0.05, 2), 3)
        return (lambda e: a(e) * c), (lambda e: an(e) * c)
    if kind == "div":
        c = round(rng.uniform(0.5, 12), 3)
        return (lambda e: a(e) / c), (lambda e: an(e) / c)
    f, fn = _score_free(rng, 2)
    if kind == "add":
        return (lambda e: a(e) + f(e)), (lambda e: an(e) + fn(e))
    if kind == "radd":
        return (lambda e: f(e) + a(e)), (lambda e: fn(e) + an(e))
    if kind == "sub":
        return (lambda e: a(e) - f(e)), (lambda e: an(e) - fn(e))
    c = round(rng.uniform(0.1, 2), 3)
    return (lambda e: (a(e) + f(e)) * c), (lambda e: (an(e) + fn(e)) * c)


def _value_of(form, s, q, k):
    x = s * form.scale + form.bias + (VALUE[form.bias_tensor] if form.bias_tensor else 0.0)
    for mono, coef in form.extra.items():
        v = coef
        for f in mono:
            v *= {"i:q_idx": q, "i:kv_idx": k}.get(f, VALUE.get(f[2:]))
        x += v
    if form.softcap is not None:
        x = form.softcap * math.tanh(x)
    return {"sigmoid": 1 / (1 + math.exp(-x)), "relu": max(x, 0.0), "identity": x}[form.activation]


@pytest.mark.parametrize("first_seed", range(0, 1500, 100))
def test_canonical_form_takes_the_expression_s_value(first_seed):
    for seed in range(first_seed, first_seed + 100):
        rng = random.Random(seed)
        a, an = _affine(rng, rng.randint(0, 4))
        act, cap = rng.choice(["none", "none", "sigmoid by tanh", "softcap", "relu", "sigmoid"]), round(rng.uniform(1, 50), 2)

        def score_mod(s, c, b, h, q, k):
            x = a({"s": s, "q": q, "k": k})
            return {"none": lambda: x, "sigmoid by tanh": lambda: (x * 0.5).tanh() * 0.5 + 0.5, "softcap": lambda: x.tanh() * cap,
                    "relu": lambda: x.max(0), "sigmoid": lambda: 1 / (1 + (-x).exp())}[act]()

        def value(s, q, k):
            x = an({"s": s, "q": q, "k": k})
            return {"none": x, "sigmoid by tanh": 1 / (1 + math.exp(-x)), "softcap": cap * math.tanh(x), "relu": max(x, 0.0),
                    "sigmoid": 1 / (1 + math.exp(-x))}[act]

        form = canonicalize_score_mod(score_mod, IO)
        for _ in range(6):
            s, q, k = rng.uniform(-8, 8), rng.randint(0, 500), rng.randint(0, 500)
            want, got = value(s, q, k), _value_of(form, s, q, k)
            assert abs(want - got) <= 1e-6 * max(1.0, abs(want)), (seed, act, form)
