"""``patch_hf`` (inf_llm/utils/patch.py:33-172) for the decoder classes of the installed transformers release.

What the patch establishes is the reference's contract (patch.py:5-31, 98-115): every attention module calls
``forward(self, hidden, hidden, rope, use_cache, past, q_proj, k_proj, v_proj, o_proj, head_dim, heads,
kv_heads)`` of the chosen attention type and gets back ``(output, cache)``; the model hands
``past_key_values[i]`` to layer i and returns the tuple of the layers' caches as ``past_key_values``, one object
per layer (a ``ContextManager`` for "inf-llm").  The model's own rotary embedding, attention mask and cache
classes are bypassed: positions are the attention type's business.

How it is wired differs from the reference because the library's classes changed: decoder layers no longer return
their cache and attention modules have no ``rotary_emb`` / ``num_heads`` attributes.  The patched attention
``forward`` therefore takes its layer's cache from, and leaves the new one on, the module itself, where the
patched model ``forward`` puts and collects them; RoPE base and head counts come from the config.
"""
import types

from ..attention import ATTN_FORWRAD, RotaryEmbeddingESM


def _rope_base(config):
    params = getattr(config, "rope_parameters", None)
    if isinstance(params, dict) and params.get("rope_theta") is not None:
        return params["rope_theta"]
    theta = getattr(config, "rope_theta", None)
    if theta is None:
        raise ValueError("the model config names no rope_theta; pass base=... to patch_hf")
    return theta


def _attention_forward(forward):
    def hf_forward(self, hidden_states, *args, **kwargs):
        assert not kwargs.get("output_attentions", False)
        cfg = self.config
        use_cache = self._infllm_use_cache
        ret = forward(self, hidden_states, hidden_states, self._infllm_rope, use_cache, self._infllm_past,
                      self.q_proj, self.k_proj, self.v_proj, self.o_proj, self.head_dim,
                      cfg.num_attention_heads, cfg.num_key_value_heads)
        if use_cache:
            out, self._infllm_new = ret
        else:
            out, self._infllm_new = ret, None
        return out, None
    return hf_forward


def _model_forward(self, input_ids=None, attention_mask=None, position_ids=None, past_key_values=None,
                   inputs_embeds=None, use_cache=None, output_attentions=None, output_hidden_states=None,
                   return_dict=None, *args, **kwargs):
    from transformers.modeling_outputs import BaseModelOutputWithPast
    assert not output_attentions
    use_cache = use_cache if use_cache is not None else self.config.use_cache
    if (input_ids is None) == (inputs_embeds is None):
        raise ValueError("pass exactly one of input_ids and inputs_embeds")
    if inputs_embeds is None:
        inputs_embeds = self.embed_tokens(input_ids)
        if hasattr(self.config, "scale_emb"):
            inputs_embeds = inputs_embeds * self.config.scale_emb
    hidden = inputs_embeds
    caches = ()
    every = () if output_hidden_states else None
    for i, layer in enumerate(self.layers):
        if every is not None:
            every += (hidden,)
        attn = layer.self_attn
        attn._infllm_past = past_key_values[i] if past_key_values is not None else None
        attn._infllm_use_cache = bool(use_cache)
        hidden = layer(hidden)
        if isinstance(hidden, tuple):
            hidden = hidden[0]
        if use_cache:
            caches += (attn._infllm_new,)
        attn._infllm_past = attn._infllm_new = None
    hidden = self.norm(hidden)
    if every is not None:
        every += (hidden,)
    if return_dict is False:
        return tuple(v for v in (hidden, caches if use_cache else None, every) if v is not None)
    return BaseModelOutputWithPast(last_hidden_state=hidden, past_key_values=caches if use_cache else None,
                                   hidden_states=every, attentions=None)


def patch_hf(model, attn_type: str = "inf-llm", attn_kwargs: dict = {}, base=None, distance_scale=None, **kwargs):
    attn_kwargs = dict(attn_kwargs)
    attn_kwargs.update(kwargs)
    if attn_type == "inf_llm":                      # the reference's default spelling is not a registry key
        attn_type = "inf-llm"
    inner = getattr(model, "model", None)
    layers = getattr(inner, "layers", None)
    if inner is None or layers is None or not hasattr(layers[0], "self_attn"):
        raise ValueError("patch_hf expects a decoder-only causal LM with model.layers[i].self_attn "
                         "(Llama, Mistral, Qwen2 and models built like them)")
    first = layers[0].self_attn
    for name in ("q_proj", "k_proj", "v_proj", "o_proj", "head_dim"):
        if not hasattr(first, name):
            raise ValueError(f"attention module {type(first).__name__} has no attribute {name}")
    device = next(model.parameters()).device
    rope = RotaryEmbeddingESM(first.head_dim, base if base is not None else _rope_base(model.config),
                              distance_scale if distance_scale is not None else 1.0, device=device)
    inner.position_bias = rope
    forward = _attention_forward(ATTN_FORWRAD[attn_type](**attn_kwargs))
    for layer in layers:
        attn = layer.self_attn
        attn._old_forward = attn.forward
        attn._infllm_rope = rope
        attn._infllm_past = attn._infllm_new = None
        attn._infllm_use_cache = True
        attn.forward = types.MethodType(forward, attn)
    inner._old_forward = inner.forward
    inner.forward = types.MethodType(_model_forward, inner)
    return model
