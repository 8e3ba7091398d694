"""Oracle: multi-stage dot-product attention with one joint softmax (test infrastructure only).

Restates TorchMultiStageDotProductionAttention
(inf_llm/attention/dot_production_attention/torch_impl.py:6-96, base.py:3-30).

Stage masks (torch_impl.py:60-78), with i the query row, j the key column:
    none                       -> every (i, j) visible
    int w                      -> (offset, size) = (len_k - len_q, w)
    (offset, size), normal     -> 0 <= i - j + offset < size
    (offset, size), complement -> i - j + offset >= size
Logits are q.k^T, masked to -inf, then scaled by 1/sqrt(D) (torch_impl.py:86-93).
At ``end`` all stages' logits are concatenated along the key axis and go
through ONE softmax (torch_impl.py:15-17); a stage's output contribution is its
slice of the probabilities (masked entries forced to 0) times its values, and
its score is the column sum of that slice over the queries (torch_impl.py:19-36).
K/V with fewer heads are repeated group-wise: head h reads kv head
h // (H / Hkv) (torch_impl.py:50-58).
"""
import math
import torch


def stage_mask(len_q, len_k, sliding_window=None, complement=False):
    """Boolean [len_q, len_k] visibility matrix of one stage."""
    if sliding_window is None:
        return torch.ones(len_q, len_k, dtype=torch.bool)
    if isinstance(sliding_window, int):
        offset, size = len_k - len_q, sliding_window
    else:
        offset, size = sliding_window
    i = torch.arange(len_q, dtype=torch.int64)[:, None]
    j = torch.arange(len_k, dtype=torch.int64)[None, :]
    dist = i - j + offset
    return dist >= size if complement else (dist >= 0) & (dist < size)


def expand_kv(x, num_heads):
    """[B, Hkv, L, D] -> [B, H, L, D], head h <- kv head h // (H/Hkv)."""
    hkv = x.shape[1]
    if hkv == num_heads:
        return x
    return x.repeat_interleave(num_heads // hkv, dim=1)


class MultiStageOracle:
    def __init__(self, q_shape, dtype=torch.float32, device="cpu"):
        self.q_shape = tuple(q_shape)
        self.dtype = dtype
        self._stages = []       # (scaled masked logits, mask, values, want_score)
        self.ret = None
        self.score_list = []

    def append(self, q, k, v, sliding_window=None, complement_sliding_window=False,
               end=False, get_score=False):
        heads = q.shape[1]
        k = expand_kv(k, heads)
        v = expand_kv(v, heads)
        mask = stage_mask(q.shape[-2], k.shape[-2], sliding_window, complement_sliding_window)
        logits = q @ k.transpose(-1, -2)
        logits = logits.masked_fill(~mask, float("-inf")) * (1.0 / math.sqrt(q.shape[-1]))
        self._stages.append((logits, mask, v, get_score))
        if end:
            self._finish()

    def _finish(self):
        p = torch.softmax(torch.cat([s[0] for s in self._stages], dim=-1), dim=-1)
        out = torch.zeros(self.q_shape, dtype=self.dtype)
        col = 0
        for logits, mask, v, want_score in self._stages:
            width = logits.shape[-1]
            ps = p[..., col:col + width].masked_fill(~mask, 0)
            self.score_list.append(ps.sum(dim=-2) if want_score else None)
            out += ps @ v
            col += width
        self.ret = out

    def get_result(self):
        return self.ret, self.score_list
