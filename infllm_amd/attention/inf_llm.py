"""The "inf-llm" attention type: factory with the signature and defaults of
inf_llm/attention/inf_llm.py:5-77.  The returned ``forward`` is what a patched
decoder layer calls; the ContextManager it creates is the layer's KV-cache
object and is handed back to the caller, as in the reference."""
from typing import Optional

import torch

from .context_manager import ContextManager


def inf_llm_forward(n_local, n_init, topk, block_size, max_cached_block, exc_block_size, fattn,
                    repr_topk: int = 1, cache_strategy="lru", score_decay=None, chunk_topk_calc=None,
                    async_global_stream=True, pin_memory=False, faiss=False, perhead=False, *args, **kwargs):

    def forward(self, query: torch.Tensor, key_value: torch.Tensor, position_bias: Optional[torch.Tensor],
                use_cache: bool, past_key_value, project_q, project_k, project_v, attention_out,
                dim_head, num_heads, num_heads_kv):
        batch_size, len_q, len_k = query.size(0), query.size(1), key_value.size(1)
        assert use_cache

        # [B, L, heads*dim] -> [B, heads, L, dim] as strided views: the prologue kernel reads
        # them in place, so the three permute copies of inf_llm.py:40-42 are not made
        h_q = project_q(query).view(batch_size, len_q, num_heads, dim_head).permute(0, 2, 1, 3)
        h_k = project_k(key_value).view(batch_size, len_k, num_heads_kv, dim_head).permute(0, 2, 1, 3)
        h_v = project_v(key_value).view(batch_size, len_k, num_heads_kv, dim_head).permute(0, 2, 1, 3)

        if past_key_value is None:
            past_key_value = ContextManager(
                position_bias, n_init, n_local, block_size, max_cached_block, topk, exc_block_size,
                score_decay, fattn, repr_topk, cache_strategy, chunk_topk_calc, async_global_stream,
                pin_memory, faiss, perhead)

        o = past_key_value.append(h_q, h_k, h_v, h_q, h_k, h_v)

        o = o.view(batch_size, num_heads, len_q, dim_head).permute(0, 2, 1, 3)
        o = attention_out(o.reshape(batch_size, len_q, dim_head * num_heads))
        if use_cache:
            return o, past_key_value
        return o

    return forward
