"""Shared body of the attention types that keep attention sinks plus a sliding window
("stream-llm", "infinite-lm": inf_llm/attention/stream_llm.py:6-111, infinite_lm.py:6-100) and of
plain causal attention ("origin": origin.py:4-79), on the multi-stage HIP operator.

The reference re-rotates the whole cached window on every call (positions relative to the window).
Here every key is rotated once, at its absolute stream position, when it arrives, and the cache keeps
the rotated rows: q.k then depends on the position difference only, which is what the window-relative
tables produce.  The sink stage uses one fixed query angle:

  infinite-lm   query at position n_local - 1, sink keys un-rotated        (infinite_lm.py:59-66)
  stream-llm    query at position n_local + n_init - 1, sink key j at j     (stream_llm.py:62-73)

A sink key j is visible to the query at stream position p in that stage iff p - j >= n_local (otherwise it
is still inside the window and the local stage sees it).  The cache tuple keeps the reference's first three
fields (keys, values, tokens seen); a fourth holds the un-rotated sink keys when the type needs them.
"""
import torch

from .. import ops
from ._rows import check_head_dim, narrow, wide_inv_freq, widen
from .dot_production_attention import get_multi_stage_dot_production_attention


def _heads(x, batch, length, heads, dim):
    return x.view(batch, length, heads, dim).permute(0, 2, 1, 3)


def _rope_args(position_bias, device):
    return wide_inv_freq(position_bias.inv_freq, device), float(position_bias.distance_scale)


def _rope(x, inv_freq, scale, pos0, consecutive=True):
    """rows rotated at pos0 + r (or all at pos0); narrower heads take the way through a 128-wide row"""
    d = x.shape[-1]
    if d == ops.HEAD_DIM:
        return ops.rope_rows(x, inv_freq, scale, pos0, consecutive)
    check_head_dim(d)
    return narrow(ops.rope_rows(widen(x, d), inv_freq, scale, pos0, consecutive), d).contiguous()


def sink_window_forward(kind, n_local, n_init, fattn=False):
    assert kind in ("stream-llm", "infinite-lm")
    Attn, _ = get_multi_stage_dot_production_attention(fattn)
    sink_query_pos = n_local - 1 if kind == "infinite-lm" else n_local + n_init - 1
    raw_sinks = kind == "infinite-lm"

    def forward(self, query, key_value, position_bias, use_cache, past_key_value, project_q, project_k, project_v,
                attention_out, dim_head, num_heads, num_heads_kv):
        batch, len_q, len_new = query.size(0), query.size(1), key_value.size(1)
        q = _heads(project_q(query), batch, len_q, num_heads, dim_head)
        k = _heads(project_k(key_value), batch, len_new, num_heads_kv, dim_head)
        v = _heads(project_v(key_value), batch, len_new, num_heads_kv, dim_head)
        if q.dtype != torch.bfloat16:
            raise TypeError(f"the HIP attention path computes in bfloat16, got {q.dtype}")
        inv_freq, scale = _rope_args(position_bias, q.device)

        seen = past_key_value[2] if past_key_value is not None else 0
        len_k = seen + len_new
        q_loc = _rope(q, inv_freq, scale, len_k - len_q)
        k_rot = _rope(k, inv_freq, scale, seen)
        v_all = v
        sinks = None
        if past_key_value is not None:
            k_rot = torch.cat((past_key_value[0], k_rot), dim=2)
            v_all = torch.cat((past_key_value[1], v), dim=2)
            sinks = past_key_value[3]
        if raw_sinks:                                       # un-rotated copies of the first n_init keys
            have = 0 if sinks is None else sinks.size(2)
            if have < n_init and seen == have:
                fresh = k[:, :, :n_init - have]
                sinks = fresh.contiguous() if sinks is None else torch.cat((sinks, fresh), dim=2)

        rows = k_rot.size(2)                                # all tokens, or n_init sinks followed by the tail
        if use_cache:
            if len_k <= n_local + n_init:
                cache = (k_rot, v_all, len_k, sinks)
            else:
                cut = max(0, rows - n_local)
                cache = (torch.cat((k_rot[:, :, :n_init], k_rot[:, :, cut:]), dim=2),
                         torch.cat((v_all[:, :, :n_init], v_all[:, :, cut:]), dim=2), len_k, sinks)
        else:
            cache = None

        first = max(0, rows - len_q - n_local)              # the local stage never needs more than this tail
        attn = Attn(q_loc.shape, q_loc.dtype, q_loc.device)
        attn.append(q_loc, k_rot[:, :, first:], v_all[:, :, first:], sliding_window=n_local)
        if len_k > n_local:
            q_sink = _rope(q, inv_freq, scale, sink_query_pos, consecutive=False)
            k_sink = sinks if raw_sinks and sinks is not None else k_rot[:, :, :n_init]
            v_sink = v_all[:, :, :n_init]
        else:
            q_sink = q.contiguous()
            k_sink = k_rot[:, :, :0]
            v_sink = v_all[:, :, :0]
        attn.append(q_sink, k_sink, v_sink, end=True, sliding_window=(len_k - len_q, n_local),
                    complement_sliding_window=True)
        o, _ = attn.get_result()

        o = o.view(batch, num_heads, len_q, dim_head).permute(0, 2, 1, 3).reshape(batch, len_q, num_heads * dim_head)
        o = attention_out(o)
        return (o, cache) if use_cache else o

    return forward


def causal_forward(fattn=False):
    Attn, _ = get_multi_stage_dot_production_attention(fattn)

    def forward(self, query, key_value, position_bias, use_cache, past_key_value, project_q, project_k, project_v,
                attention_out, dim_head, num_heads, num_heads_kv):
        assert use_cache                                                           # origin.py:18
        batch, len_q, len_new = query.size(0), query.size(1), key_value.size(1)
        q = _heads(project_q(query), batch, len_q, num_heads, dim_head)
        k = _heads(project_k(key_value), batch, len_new, num_heads_kv, dim_head)
        v = _heads(project_v(key_value), batch, len_new, num_heads_kv, dim_head)
        if q.dtype != torch.bfloat16:
            raise TypeError(f"the HIP attention path computes in bfloat16, got {q.dtype}")
        inv_freq, scale = _rope_args(position_bias, q.device)
        seen = past_key_value[0].size(2) if past_key_value is not None else 0
        len_k = seen + len_new
        q_rot = _rope(q, inv_freq, scale, len_k - len_q)
        k_rot = _rope(k, inv_freq, scale, seen)
        v_all = v.contiguous()
        if past_key_value is not None:
            k_rot = torch.cat((past_key_value[0], k_rot), dim=2)
            v_all = torch.cat((past_key_value[1], v_all), dim=2)
        attn = Attn(q_rot.shape, q_rot.dtype, q_rot.device)
        attn.append(q_rot, k_rot, v_all, sliding_window=len_k, end=True)          # window >= everything: causal
        o, _ = attn.get_result()
        o = o.view(batch, num_heads, len_q, dim_head).permute(0, 2, 1, 3).reshape(batch, len_q, dim_head * num_heads)
        return attention_out(o), (k_rot, v_all)

    return forward
