"""MI355X-native backend for the MetaAttention ``attention_engine`` API.

The reference is used with its ``attention_engine/`` directory on PYTHONPATH so
that user specs can ``from attn_engine import AttentionEngine`` and ``from core
import SymbolScalar`` (docker/Dockerfile.rocm:25 of the reference).  Importing
this package puts its own directory on ``sys.path`` so the same top-level names
(``attn_engine``, ``core``, ``autotuner``) resolve to this implementation.
"""
import os
import sys

_HERE = os.path.dirname(os.path.abspath(__file__))
if _HERE not in sys.path:
    sys.path.insert(0, _HERE)

from attn_engine import AttentionEngine, LinearAttentionEngine, OnlineFunc  # noqa: E402,F401
from core import CustomIO, SymbolicArray, SymbolScalar, SymbolicTensor, Var, meta_tensor  # noqa: E402,F401
from autotuner.arch import get_attn_device  # noqa: E402,F401
