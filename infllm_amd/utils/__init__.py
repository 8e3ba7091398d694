"""Model-side glue with the names of inf_llm/utils/__init__.py: ``patch_hf`` routes the attention of a
Hugging Face decoder through an attention type of this package, ``GreedySearch`` is the chunked-prefill
greedy generation driver."""
from .patch import patch_hf
from .greedy_search import GreedySearch

__all__ = ["patch_hf", "GreedySearch"]
