from .transform.core import CustomIO, SymbolicArray, SymbolScalar, SymbolicTensor, SymbolicConst, Var
from .utils import meta_tensor
