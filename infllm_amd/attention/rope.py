"""RotaryEmbeddingESM with the interface of inf_llm/attention/rope.py:4-112.

The streaming path does not call ``forward`` / ``apply_rotary_pos_emb_one_angle``:
RoPE is fused into the prologue kernel (infllm_ingest), which only needs this
module's ``inv_freq`` (fp32, computed exactly like rope.py:22-24), ``base`` and
``distance_scale``.  The tensor methods are kept, with the reference's
semantics, for callers that rotate tensors themselves (the sibling attention
types do): fp32 math, half-split pairing, result cast back to the input dtype.
"""
import torch


class RotaryEmbeddingESM(torch.nn.Module):
    def __init__(self, dim, base=10000, distance_scale=1, device=None):
        super().__init__()
        self.dim = dim
        self.base = base
        self.distance_scale = distance_scale
        if device is None:
            device = "cuda" if torch.cuda.is_available() else "cpu"
        exponent = torch.arange(0, dim, 2, device=device, dtype=torch.float32) / dim
        self.register_buffer("inv_freq", 1.0 / (base ** exponent), persistent=False)
        self._seq_len_cached = -1
        self._cos_cached = None
        self._sin_cached = None

    # ---- tables -----------------------------------------------------------
    def _build(self, seq_len, device, ndim):
        t = torch.arange(seq_len, device=device).type_as(self.inv_freq)
        ang = torch.outer(t * self.distance_scale, self.inv_freq.to(device))
        ang = torch.cat((ang, ang), dim=-1)
        shape = (1,) * (ndim - 2) + tuple(ang.shape)
        self._seq_len_cached = seq_len
        self._cos_cached, self._sin_cached = ang.cos().view(shape), ang.sin().view(shape)

    def _update_cos_sin_tables(self, x, seq_dim=-2):
        if x.size(seq_dim) > self._seq_len_cached:
            self._build(x.size(seq_dim), x.device, x.dim())
        return self._cos_cached, self._sin_cached

    def _update_cos_sin_tables_len(self, seq_len, device, dim=None):
        if seq_len > self._seq_len_cached:
            if dim is None:
                assert self._cos_cached is not None
                dim = self._cos_cached.dim()
            self._build(seq_len, device, dim)
        return self._cos_cached, self._sin_cached

    # ---- application ------------------------------------------------------
    @staticmethod
    def rotate_half(x):
        half = x.shape[-1] // 2
        return torch.cat((-x[..., half:], x[..., :half]), dim=-1)

    def apply_rotary_pos_emb(self, x, length, right, cos, sin):
        cos, sin = cos[..., right - length:right, :], sin[..., right - length:right, :]
        return (x.float() * cos + self.rotate_half(x).float() * sin).to(x.dtype)

    def apply_rotary_pos_emb_one_angle(self, x, index):
        cos, sin = self._update_cos_sin_tables_len(index, x.device, x.dim())
        cos, sin = cos[..., index - 1:index, :], sin[..., index - 1:index, :]
        return (x.float() * cos + self.rotate_half(x).float() * sin).to(x.dtype)

    def forward(self, q, k, seq_dim=-2):
        cos, sin = self._update_cos_sin_tables(k, seq_dim=seq_dim)
        return (self.apply_rotary_pos_emb(q, q.size(seq_dim), k.size(seq_dim), cos, sin),
                self.apply_rotary_pos_emb(k, k.size(seq_dim), k.size(seq_dim), cos, sin))
