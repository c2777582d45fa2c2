"""Top-level ``attn_engine`` package (same exports as the reference's
attention_engine/attn_engine/__init__.py:1-2, minus the linear-attention engine, which is a
different algorithm and not part of this build)."""
from .attn_engine import AttentionEngine, OnlineFunc

__all__ = ["AttentionEngine", "OnlineFunc"]
