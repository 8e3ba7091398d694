"""Model-side glue with the names of inf_llm/utils/__init__.py: ``patch_hf`` routes the attention of a
Hugging Face decoder through an attention type of this package, ``GreedySearch`` is the chunked-prefill
greedy generation driver; ``load_config`` reads the reference's YAML run configurations."""
from .patch import patch_hf
from .greedy_search import GreedySearch
from .config import load_config, patch_from_config

__all__ = ["patch_hf", "GreedySearch", "load_config", "patch_from_config"]
