"""Oracle: the "inf-llm" attention type backed by oracle.stream on the CPU (test infrastructure only).

Restates inf_llm/attention/inf_llm.py:5-77 with StreamOracle in place of ContextManager, so that a decoder
patched with it is the fp32 CPU counterpart of the same decoder patched with the product's attention type.
"""
from .rope import RopeOracle
from .stream import StreamOracle


def oracle_inf_llm_forward(n_local, n_init, topk, block_size, max_cached_block, exc_block_size, fattn=False,
                           repr_topk=1, cache_strategy="lru", score_decay=None, chunk_topk_calc=None,
                           async_global_stream=True, pin_memory=False, faiss=False, perhead=False, *args, **kwargs):
    def forward(self, query, key_value, position_bias, use_cache, past_key_value, project_q, project_k, project_v,
                attention_out, dim_head, num_heads, num_heads_kv):
        assert use_cache                                                       # inf_llm.py:33
        batch, len_q, len_k = query.size(0), query.size(1), key_value.size(1)
        heads = lambda x, n, h: x.view(batch, n, h, dim_head).permute(0, 2, 1, 3).contiguous().float()
        q = heads(project_q(query), len_q, num_heads)                          # :36-42
        k = heads(project_k(key_value), len_k, num_heads_kv)
        v = heads(project_v(key_value), len_k, num_heads_kv)
        if past_key_value is None:                                             # :44-58
            rope = RopeOracle(dim_head, base=position_bias.base, distance_scale=position_bias.distance_scale)
            past_key_value = StreamOracle(rope, n_init, n_local, block_size, max_cached_block, topk, exc_block_size,
                                          score_decay=score_decay, repr_topk=repr_topk, cache_strategy=cache_strategy,
                                          perhead=perhead, chunk_topk_calc=chunk_topk_calc)
        o = past_key_value.append(q, k, v)                                     # :60-66
        o = o.view(batch, num_heads, len_q, dim_head).permute(0, 2, 1, 3).reshape(batch, len_q, dim_head * num_heads)
        return attention_out(o.to(query.dtype)), past_key_value                # :68-77
    return forward
