"""Multi-stage attention on the gfx950 MFMA kernel.

Same call protocol as TorchMultiStageDotProductionAttention /
TritonMultiStageDotProductionAttention
(inf_llm/attention/dot_production_attention/torch_impl.py:6-96,
triton_impl.py:488-556): every ``append`` is one stage with its own keys,
values and sliding-window mask; ``end=True`` closes the joint softmax;
``get_result()`` returns the output and, per stage, the column sums of the
final probabilities (or None).  Each stage is one launch of infllm_attn_stage
that leaves a partial (o, lse); the merge kernel joins them, and the scores
are computed afterwards from the final lse (infllm_local_score).  Scores are
returned in fp32.  Heads narrower than 128 are padded with zeros to the kernels'
width (the softmax scale stays 1/sqrt of the real head_dim) and the result is cut
back.
"""
import math

import torch
import torch.nn.functional as F

from ... import ops
from .base import MultiStageDotProductionAttention


class HipMultiStageDotProductionAttention(MultiStageDotProductionAttention):
    def __init__(self, q_shape, dtype, device):
        super().__init__(q_shape, dtype, device)
        if dtype != torch.bfloat16:
            raise TypeError(f"the HIP attention path computes in bfloat16, got {dtype}")
        self._stages = []          # (q, k, mask, offset, window, get_score)
        self._o_parts = []
        self._lse_parts = []

    def append(self, q, k, v, sliding_window=None, complement_sliding_window=False, end=False, get_score=False,
               *args, **kwargs):
        assert tuple(q.shape) == self.q_shape
        assert not self.end, "append after end"
        d = q.shape[-1]
        if d < ops.HEAD_DIM:
            q, k, v = (F.pad(t, (0, ops.HEAD_DIM - d)) for t in (q, k, v))
        q, k, v = ops._bf16_4d(q, "q"), ops._bf16_4d(k, "k"), ops._bf16_4d(v, "v")
        B, H, Lq, D = q.shape
        scale = 1.0 / math.sqrt(d)
        len_k = k.shape[2]
        if sliding_window is None:
            mask, offset, window = ops.MASK_NONE, 0, 0
        else:
            if isinstance(sliding_window, int):
                sliding_window = (len_k - Lq, sliding_window)
            offset, window = int(sliding_window[0]), int(sliding_window[1])
            mask = ops.MASK_COMPLEMENT if complement_sliding_window else ops.MASK_WINDOW
        o_part = torch.empty((1, B, H, Lq, D), dtype=torch.float16, device=q.device)
        lse_part = torch.empty((1, B, H, Lq), dtype=torch.float32, device=q.device)
        ops.attn_stage_linear(q, k, v, o_part, lse_part, j_lo=0, j_hi=len_k, mask=mask, offset=offset, window=window, softmax_scale=scale)
        self._o_parts.append(o_part)
        self._lse_parts.append(lse_part)
        self._stages.append((q, k, mask, offset, window, get_score, scale))
        if end:
            self._finalize()

    def _finalize(self):
        self.end = True
        B, H, Lq, d = self.q_shape
        D = max(d, ops.HEAD_DIM)
        P = len(self._stages)
        o_all = torch.cat(self._o_parts, dim=0) if P > 1 else self._o_parts[0]
        lse_all = torch.cat(self._lse_parts, dim=0) if P > 1 else self._lse_parts[0]
        dev = o_all.device
        self.ret = torch.empty((B, H, Lq, D), dtype=torch.bfloat16, device=dev)
        self.lse = torch.empty((B, H, Lq), dtype=torch.float32, device=dev)
        ops.attn_merge(o_all, lse_all, P, self.ret, self.lse)
        if d < D:
            self.ret = self.ret[..., :d].contiguous()
        for q, k, mask, offset, window, want, scale in self._stages:
            if not want:
                self.score_list.append(None)
                continue
            score = torch.zeros((B, H, k.shape[2]), dtype=torch.float32, device=dev)
            if k.shape[2] > 0:
                ops.local_score(q, k, self.lse, score, j_lo=0, j_hi=k.shape[2], mask=mask, offset=offset,
                                window=window, accumulate=False, softmax_scale=scale)
            self.score_list.append(score)
        self._o_parts, self._lse_parts = [], []
