"""The "origin" attention type (inf_llm/attention/origin.py:4): plain causal attention with RoPE and a growing
key/value cache; factory signature of the reference."""
from ._sink_window import causal_forward


def origin_forward(fattn: bool, *args, **kwargs):
    return causal_forward(fattn)
