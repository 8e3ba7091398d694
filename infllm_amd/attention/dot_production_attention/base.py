"""Operator interface of the multi-stage attention
(inf_llm/attention/dot_production_attention/base.py:3-30)."""


class MultiStageDotProductionAttention:
    """Stages appended one by one share ONE softmax; see the HIP implementation."""

    def __init__(self, q_shape, dtype, device):
        self.q_shape = tuple(q_shape)
        self.dtype = dtype
        self.device = device
        self.end = False
        self.ret = None
        self.score_list = []

    def append(self, q, k, v, sliding_window=None, complement_sliding_window=False, end=False, get_score=False,
               *args, **kwargs):
        raise NotImplementedError

    def get_result(self):
        return self.ret, self.score_list
