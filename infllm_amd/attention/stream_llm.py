"""The "stream-llm" attention type (inf_llm/attention/stream_llm.py:6): attention sinks rotated at their own
positions plus a sliding window; factory signature of the reference."""
from ._sink_window import sink_window_forward


def stream_llm_forward(n_local, n_init, fattn: bool = False, *args, **kwargs):
    return sink_window_forward("stream-llm", n_local, n_init, fattn)
