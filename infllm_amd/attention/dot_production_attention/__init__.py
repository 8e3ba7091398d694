"""Selector with the signature of
inf_llm/attention/dot_production_attention/__init__.py:4-26.

The reference picks between a torch and a Triton implementation; this package
has a single implementation (the HIP kernels), returned for either value of
``flash_attn``.  The second element reports that a flash-style kernel is in use.
"""
from typing import Tuple

from .base import MultiStageDotProductionAttention


def get_multi_stage_dot_production_attention(flash_attn=False) -> Tuple[type, bool]:
    from .hip_impl import HipMultiStageDotProductionAttention
    return HipMultiStageDotProductionAttention, True
