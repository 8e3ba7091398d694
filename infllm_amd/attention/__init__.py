"""Attention-type registry (inf_llm/attention/__init__.py:8-13).  The registry
name keeps the reference's spelling."""
from .rope import RotaryEmbeddingESM
from .context_manager import ContextManager
from .inf_llm import inf_llm_forward
from .infinite_lm import infinite_lm_forward
from .stream_llm import stream_llm_forward
from .origin import origin_forward

ATTN_FORWRAD = {
    "inf-llm": inf_llm_forward,
    "infinite-lm": infinite_lm_forward,
    "stream-llm": stream_llm_forward,
    "origin": origin_forward,
}

__all__ = ["RotaryEmbeddingESM", "ContextManager", "ATTN_FORWRAD", "inf_llm_forward", "infinite_lm_forward",
           "stream_llm_forward", "origin_forward"]
