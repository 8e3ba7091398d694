"""Oracle: the sink + sliding-window attention types and plain causal attention (test infrastructure only).

``SinkWindowOracle`` restates the per-call algorithm of inf_llm/attention/stream_llm.py:17-108 and
infinite_lm.py:17-97 in fp32 on the CPU, with the reference's structure: the cache is the tuple
(keys, values, tokens seen) holding un-rotated rows, truncated to the first n_init and the last n_local
tokens (:44-52); the window is re-rotated relative to itself on every call (:65); the sink stage rotates the
query by one angle and masks with the complement window at offset len_k - len_q (:68-103).
``CausalOracle`` restates origin.py:12-77.

``sink_window_dense`` is NOT a restatement: it derives the same result for a whole stream at once from
absolute positions (one dense softmax per query over window keys and visible sinks) and pins the class above
(tests/test_oracle_siblings.py), together with the reductions to causal / banded SDPA.
"""
import torch

from .multistage import MultiStageOracle


class SinkWindowOracle:
    def __init__(self, rope, n_local, n_init, kind):
        assert kind in ("stream-llm", "infinite-lm")
        self.rope, self.n_local, self.n_init, self.kind = rope, n_local, n_init, kind
        self.cache = None

    def append(self, q, k, v):
        """q [B,H,L,D], k/v [B,Hkv,L,D] of the new tokens -> [B,H,L,D]."""
        n_local, n_init = self.n_local, self.n_init
        len_q, len_k = q.shape[2], k.shape[2]
        if self.cache is not None:                                          # :37-41
            k = torch.cat((self.cache[0], k), dim=2)
            v = torch.cat((self.cache[1], v), dim=2)
            len_k += self.cache[2]
        if len_k <= n_local + n_init:                                       # :43-52
            self.cache = (k, v, len_k)
        else:
            cut = max(0, k.shape[2] - n_local)
            self.cache = (torch.cat((k[:, :, :n_init], k[:, :, cut:]), dim=2),
                          torch.cat((v[:, :, :n_init], v[:, :, cut:]), dim=2), len_k)
        wk, wv = k, v
        if len_q + n_local < k.shape[2]:                                    # :61-63
            wk, wv = k[:, :, k.shape[2] - len_q - n_local:], v[:, :, v.shape[2] - len_q - n_local:]
        q_rot, k_rot = self.rope.window(q, wk)                              # :66
        if len_k > n_local:                                                 # :69-80
            if self.kind == "stream-llm":
                sq = self.rope.one_angle(q, n_local + n_init)
                sk = self.rope.rotate(k[:, :, :n_init], range(min(n_init, k.shape[2])))
            else:
                sq = self.rope.one_angle(q, n_local)
                sk = k[:, :, :n_init]
            sv = v[:, :, :n_init]
        else:
            sq, sk, sv = q, k[:, :, :0], v[:, :, :0]
        attn = MultiStageOracle(q.shape)
        attn.append(q_rot, k_rot, wv, sliding_window=n_local)               # :95-102
        attn.append(sq, sk, sv, end=True, sliding_window=(len_k - len_q, n_local), complement_sliding_window=True)
        out, _ = attn.get_result()
        return out


class CausalOracle:
    def __init__(self, rope):
        self.rope, self.cache = rope, None

    def append(self, q, k, v):
        if self.cache is not None:                                          # origin.py:29-32
            k = torch.cat((self.cache[0], k), dim=2)
            v = torch.cat((self.cache[1], v), dim=2)
        self.cache = (k, v)
        len_q, len_k = q.shape[2], k.shape[2]
        q_rot, k_rot = self.rope.window(q, k)                               # :37
        attn = MultiStageOracle(q.shape)
        attn.append(q_rot, k_rot, v, sliding_window=len_k, end=True)        # :46-63: dist >= 0
        return attn.get_result()[0]


def sink_window_dense(q, k, v, rope, n_local, n_init, kind):
    """Whole stream at once, absolute positions.  q [H,T,D], k/v [Hkv,T,D] -> [H,T,D] (fp64).

    Query p sees key j <= p with p - j < n_local at rotary distance p - j, and sink key j < n_init with
    p - j >= n_local at the fixed distance of the type (infinite-lm: n_local - 1; stream-llm:
    n_local + n_init - 1 - j); one softmax over both sets, scale 1/sqrt(D).
    """
    H, T, D = q.shape
    G = H // k.shape[0]
    kf, vf = k.repeat_interleave(G, dim=0).double(), v.repeat_interleave(G, dim=0).double()
    pos = list(range(T))
    q_abs, k_abs = rope.rotate(q.float(), pos).double(), rope.rotate(k.float(), pos).repeat_interleave(G, dim=0).double()
    logits = torch.einsum("hpd,hjd->hpj", q_abs, k_abs)                     # relative distance p - j
    if kind == "infinite-lm":
        sq = rope.one_angle(q.float(), n_local).double()
        sink_logits = torch.einsum("hpd,hjd->hpj", sq, kf[:, :n_init])
    else:
        sq = rope.one_angle(q.float(), n_local + n_init).double()
        sink_logits = torch.einsum("hpd,hjd->hpj", sq, k_abs[:, :n_init])
    p_idx, j_idx = torch.arange(T)[:, None], torch.arange(T)[None, :]
    dist = p_idx - j_idx
    local = (dist >= 0) & (dist < n_local)
    sink = (dist >= n_local) & (j_idx < n_init)
    full = torch.full((H, T, T), float("-inf"), dtype=torch.float64)
    full = torch.where(local, logits, full)
    n_s = min(n_init, T)
    full[:, :, :n_s] = torch.where(sink[:, :n_s], sink_logits[:, :, :n_s], full[:, :, :n_s])
    prob = torch.softmax(full / D ** 0.5, dim=-1)
    return torch.einsum("hpj,hjd->hpd", prob, vf)
