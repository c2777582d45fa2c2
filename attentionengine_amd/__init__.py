"""MI355X-native implementation of AttentionEngine's fused attention path (forward, and the backward of
softmax, sigmoid and relu attention).

The reference puts ``attention_engine/`` on PYTHONPATH so that ``attn_engine``, ``core`` and
``benchmark`` are top-level packages (README.md:50) and its scripts import them by those names
(attn_script/mha.py:1-8).  Importing this package does the same for its own directory, then
re-exports the public names.
"""
import os as _os
import sys as _sys

_here = _os.path.dirname(_os.path.abspath(__file__))
if _here not in _sys.path:
    _sys.path.insert(0, _here)

from attn_engine import AttentionEngine, OnlineFunc  # noqa: E402
from core import (CustomIO, SymbolicArray, SymbolicTensor, SymbolScalar, Var,  # noqa: E402
                  create_block_mask, create_mask, meta_tensor)

__all__ = ["AttentionEngine", "OnlineFunc", "CustomIO", "SymbolicArray", "SymbolicTensor",
           "SymbolScalar", "Var", "create_block_mask", "create_mask", "meta_tensor"]
