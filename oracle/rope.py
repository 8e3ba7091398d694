"""Oracle: rotary position embedding of the reference (test infrastructure only).

Restates inf_llm/attention/rope.py:4-112 on the CPU in fp32:

* inverse frequencies ``base ** -(2i/D)`` are computed in fp32 (rope.py:22-24);
* angles are ``fp32(t * distance_scale) * inv_freq`` in fp32 (rope.py:56-57);
* the table is duplicated over both halves of the head dimension (rope.py:58)
  and pairing is half-split: element d pairs with d + D/2 (rope.py:31-33);
* math is ``x*cos + rotate_half(x)*sin`` in fp32, cast back to x's dtype
  (rope.py:47, 104).
"""
import torch


class RopeOracle:
    def __init__(self, dim, base=10000, distance_scale=1.0):
        self.dim = dim
        self.base = base
        self.distance_scale = distance_scale
        exponents = torch.arange(0, dim, 2, dtype=torch.float32) / dim
        self.inv_freq = 1.0 / (base ** exponents)          # fp32, rope.py:22-24

    def cos_sin(self, positions):
        """fp32 cos/sin rows [len(positions), dim] for integer positions."""
        t = torch.as_tensor(positions, dtype=torch.int64).to(torch.float32)
        ang = torch.outer(t * self.distance_scale, self.inv_freq)
        ang = torch.cat((ang, ang), dim=-1)
        return ang.cos(), ang.sin()

    @staticmethod
    def _swap_halves_negated(x):
        half = x.shape[-1] // 2
        return torch.cat((-x[..., half:], x[..., :half]), dim=-1)

    def rotate(self, x, positions):
        """Rotate rows of x[..., L, D]; row r sits at integer position positions[r]."""
        cos, sin = self.cos_sin(positions)
        xf = x.float()
        return (xf * cos + self._swap_halves_negated(xf) * sin).to(x.dtype)

    def window(self, q, k):
        """rope.py:107-112: keys at 0..len_k-1, queries right-aligned to the keys."""
        len_q, len_k = q.shape[-2], k.shape[-2]
        return (self.rotate(q, range(len_k - len_q, len_k)),
                self.rotate(k, range(len_k)))

    def one_angle(self, x, index):
        """rope.py:89-104: every row at position index-1."""
        return self.rotate(x, [index - 1] * x.shape[-2])
