"""Frontend package (top-level name ``core``, as in the reference: attention_engine/ is put on
PYTHONPATH, README.md:50).  Exports match attention_engine/core/__init__.py:1-2, plus
``create_block_mask`` which the reference's README imports from here (README.md:63)."""
from .transform.core import (CustomIO, SymbolicArray, SymbolicColReduceArray, SymbolicConst,
                             SymbolicTensor, SymbolScalar, Var, create_block_mask, create_mask)
from .utils import meta_tensor

__all__ = ["CustomIO", "SymbolicArray", "SymbolicColReduceArray", "SymbolicConst", "SymbolicTensor",
           "SymbolScalar", "Var", "create_block_mask", "create_mask", "meta_tensor"]
