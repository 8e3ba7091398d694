"""The "infinite-lm" attention type (inf_llm/attention/infinite_lm.py:6): un-rotated attention sinks at the
fixed distance n_local - 1 plus a sliding window; factory signature of the reference."""
from ._sink_window import sink_window_forward


def infinite_lm_forward(n_local, n_init, fattn: bool = False, *args, **kwargs):
    return sink_window_forward("infinite-lm", n_local, n_init, fattn)
