"""Operation tags of the symbolic trace.

Same closed set of node types as the reference's expression graph
(attention_engine/core/transform/graph.py:2-243): leaves ``Var`` / ``Const``,
element-wise arithmetic and transcendental ops, and row / column reductions.
A node only records its type and operands; meaning is given by the spec
interpreter (core/eager.py) and the canonicaliser (core/canonical.py).
"""
from __future__ import annotations


class Node:
    arity = 0

    def __init__(self, type: str, *inputs: "Node"):
        self.type = type
        self.inputs = list(inputs)

    def __str__(self) -> str:
        return f"{self.type}({', '.join(str(i) for i in self.inputs)})"

    __repr__ = __str__


class Var(Node):
    """Named leaf.  For row-scale state the name is the initial value as a
    string ("-inf", "0.0", "1"), exactly as user specs write it."""

    def __init__(self, name: str):
        super().__init__("Var")
        self.name = str(name)

    def __str__(self) -> str:
        return f'Var("{self.name}")'


class Const(Node):
    def __init__(self, value: float):
        super().__init__("Const")
        self.value = value

    def __str__(self) -> str:
        return f"Const({self.value})"


def _op(name: str, arity: int):
    def __init__(self, *inputs):
        if len(inputs) != arity:
            raise TypeError(f"{name} takes {arity} operand(s), got {len(inputs)}")
        Node.__init__(self, name, *inputs)
    return type(name, (Node,), {"__init__": __init__, "arity": arity})


Add, Sub, Mul, Div, Max = (_op(n, 2) for n in ("Add", "Sub", "Mul", "Div", "Max"))
Neg, Abs, Exp, Exp2, Log, Log2, Tanh = (_op(n, 1) for n in ("Neg", "Abs", "Exp", "Exp2", "Log", "Log2", "Tanh"))
MaxBwd = _op("MaxBwd", 3)
ReduceSum, ReduceMax, ReduceAbsSum = (_op(n, 1) for n in ("ReduceSum", "ReduceMax", "ReduceAbsSum"))
ColReduceSum, ColReduceMax, ColReduceAbsSum = (_op(n, 1) for n in ("ColReduceSum", "ColReduceMax", "ColReduceAbsSum"))

ELEMENTWISE_UNARY = {"Neg", "Abs", "Exp", "Exp2", "Log", "Log2", "Tanh"}
ELEMENTWISE_BINARY = {"Add", "Sub", "Mul", "Div", "Max"}
ROW_REDUCE = {"ReduceSum", "ReduceMax", "ReduceAbsSum"}
COL_REDUCE = {"ColReduceSum", "ColReduceMax", "ColReduceAbsSum"}
