"""Attention-type registry (inf_llm/attention/__init__.py:8-13).  The registry
name keeps the reference's spelling."""
from .rope import RotaryEmbeddingESM
from .context_manager import ContextManager
from .inf_llm import inf_llm_forward

ATTN_FORWRAD = {
    "inf-llm": inf_llm_forward,
}

__all__ = ["RotaryEmbeddingESM", "ContextManager", "ATTN_FORWRAD", "inf_llm_forward"]
