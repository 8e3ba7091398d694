"""Rows of heads narrower than the 128 dimensions the gfx950 kernels are built for.

MiniCPM-2B has head_dim 64 (the reference ships config/minicpm-inf-llm.yaml for it, and its operators take any
head_dim up to 128: torch_impl.py is shape-agnostic, triton_impl.py:412 lists 16 / 32 / 64 / 128).  Such rows run
on the same kernels in a 128-wide row whose unused dimensions are zero: zeros add nothing to q.k, to a
representative's score or to an output row, so only the softmax scale 1/sqrt(D) has to be the narrow head's own.

Where the kernel applies RoPE itself (the prologue, infllm_rope_rows) the two halves of a row go to dimensions
[0, D/2) and [64, 64 + D/2): the rotation pairs dimension d with d + D/2 (rope.py:31-33), which are d and d + 64 in
the wide row - the pairing the kernels use - and the frequencies of the unused slots are zero.  Twice the bytes and
flops a kernel built for 64 would need: a way to run such models, not a fast path.
"""
import torch

from ..ops import HEAD_DIM


def check_head_dim(d):
    if d > HEAD_DIM or d % 2:
        raise ValueError(f"head_dim must be even and at most {HEAD_DIM}, got {d}")


def widen(t, d):
    """[..., d] -> [..., 128] with the halves at [0, d/2) and [64, 64 + d/2)."""
    if d == HEAD_DIM:
        return t
    out = t.new_zeros(t.shape[:-1] + (HEAD_DIM,))
    out[..., :d // 2] = t[..., :d // 2]
    out[..., HEAD_DIM // 2:HEAD_DIM // 2 + d // 2] = t[..., d // 2:]
    return out


def narrow(t, d):
    """inverse of widen"""
    if d == HEAD_DIM:
        return t
    return torch.cat((t[..., :d // 2], t[..., HEAD_DIM // 2:HEAD_DIM // 2 + d // 2]), dim=-1)


def wide_inv_freq(inv_freq, device):
    """the d/2 rotary frequencies in the 64 slots of a wide row; unused slots rotate by nothing"""
    inv_freq = inv_freq.to(device=device, dtype=torch.float32)
    if inv_freq.numel() == HEAD_DIM // 2:
        return inv_freq.contiguous()
    out = torch.zeros((HEAD_DIM // 2,), dtype=torch.float32, device=device)
    out[:inv_freq.numel()] = inv_freq
    return out
