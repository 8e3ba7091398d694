"""benchmark configuration 4 at its own geometry: a decoder with the Llama-3-8B architecture (hidden 4096, 32 query / 8 kv
heads, head_dim 128, FFN 14336 SwiGLU, RoPE base 500000, vocabulary 128,256, random weights, bf16), every attention
routed through the "inf-llm" type with the reference's knobs, driven by GreedySearch with chunk_size 8192
(inf_llm/utils/greedy_search.py:52-70).

Two tests.  (i) Parity inside the model: two layers, a prompt long enough that more than topk units exist, so a real
top-k runs.  The bf16 q / k / v that each layer's ContextManager.append received are recorded and replayed through
the CPU oracle following that layer's choices (tests/stream_parity.py): attention outputs, ordered selections,
representative picks, representatives and residency events, layer by layer.  Replaying the recorded tensors keeps
the comparison on the attention path: whatever bf16 projections and MLPs do to the activations, both sides of a
layer see the same inputs.  (ii) The full-size run: 32 layers, a 131,072-token prompt, 128 greedy steps; checked
through the closed forms of the state machine, GreedySearch's call schedule and finite logits.
"""
import pytest
import torch

from stream_parity import REFERENCE, assert_tie_stats, follow

pytestmark = pytest.mark.gpu
transformers = pytest.importorskip("transformers")

H, HKV, D = 32, 8, 128
EXC, N_LOCAL, N_INIT, BS, TOPK = (REFERENCE[k] for k in ("exc_block_size", "n_local", "n_init", "block_size", "topk"))
ROPE_BASE = 500000.0
VOCAB = 128256
KNOBS = dict(REFERENCE, fattn=False)


def _llama3_8b_shape(layers, dev):
    from infllm_amd.utils import patch_hf
    cfg = transformers.LlamaConfig(hidden_size=4096, intermediate_size=14336, num_hidden_layers=layers, num_attention_heads=H,
                                   num_key_value_heads=HKV, head_dim=D, vocab_size=VOCAB, rope_theta=ROPE_BASE,
                                   max_position_embeddings=8192, tie_word_embeddings=False)
    torch.manual_seed(4)
    old = torch.get_default_dtype()
    torch.set_default_dtype(torch.bfloat16)
    try:
        with torch.device(dev):
            model = transformers.LlamaForCausalLM(cfg)
    finally:
        torch.set_default_dtype(old)
    return patch_hf(model, "inf-llm", dict(KNOBS), base=ROPE_BASE).eval()


class _Tok:
    eos_token_id = -1

    def decode(self, ids):
        return ids.tolist()


def _units_after(tokens):
    """units carved once `tokens` tokens have been consumed (context_manager.py:649-662)"""
    return max(0, (tokens - N_INIT - N_LOCAL) // BS)


def _blocks_of(calls):
    """(start position, length) of every execution block of a stream consumed in the given append() calls"""
    out, pos = [], 0
    for L in calls:
        for st in range(0, L, EXC):
            out.append((pos + st, min(EXC, L - st)))
        pos += L
    return out


def _watch_appends(monkeypatch, keep_tensors):
    """Wrap ContextManager.append: per manager (in order of first use = layer order) the call lengths, the unit count
    after every call and, if asked for, CPU copies of what went in and came out."""
    from infllm_amd.attention import ContextManager
    seen, order = {}, []
    plain = ContextManager.append

    def append(self, local_q, local_k, local_v, global_q, global_k, global_v):
        rec = seen.get(id(self))
        if rec is None:
            rec = seen[id(self)] = dict(cm=self, calls=[], units=[], q=[], k=[], v=[], o=[])
            order.append(rec)
            self.record_trace = keep_tensors
        assert global_q is local_q and global_k is local_k and global_v is local_v     # inf_llm.py:60 passes them twice
        out = plain(self, local_q, local_k, local_v, global_q, global_k, global_v)
        rec["calls"].append(local_q.shape[2])
        rec["units"].append(self.num_global_block)
        if keep_tensors:
            for name, t in (("q", local_q), ("k", local_k), ("v", local_v), ("o", out)):
                rec[name].append(t.detach().to("cpu", copy=True))
        return out

    monkeypatch.setattr(ContextManager, "append", append)
    return order


def test_config4_two_layers_at_llama3_geometry_follow_the_oracle_layer_by_layer(monkeypatch):
    from infllm_amd.utils import GreedySearch
    dev = torch.device("cuda:0")
    layers = _watch_appends(monkeypatch, keep_tensors=True)
    model = _llama3_8b_shape(2, dev)
    T, steps = 8192 + 1792 + 1, 3
    ids = torch.randint(0, VOCAB, (T,), generator=torch.Generator().manual_seed(5))
    text = GreedySearch(model, _Tok()).generate(input_ids=ids, max_length=steps, chunk_size=8192)[0]
    torch.cuda.synchronize()
    assert len(text) == steps and all(0 <= t < VOCAB for t in text)
    calls = [8192, 1792] + [1] * (1 + steps)                    # all but the last token in chunks, the last token, one per step
    assert len(layers) == 2
    for i, rec in enumerate(layers):
        cm = rec["cm"]
        assert rec["calls"] == calls, (i, rec["calls"])
        assert cm.length == T + steps and cm.num_global_block == _units_after(T + steps) > 2 * TOPK
        q, k, v, got = (torch.cat(rec[n], dim=2) for n in ("q", "k", "v", "o"))
        assert q.dtype == torch.bfloat16 and q.shape == (1, H, T + steps, D) and k.shape == (1, HKV, T + steps, D)
        # projections of random weights give q / k / v of std 1.3 reaching 7: the max-abs bound is relative beyond |o| = 1
        ora, fol = follow(cm, got, q, k, v, calls, ROPE_BASE, relative_above_one=True, **REFERENCE)
        full = [b for b in ora.block_trace if b["n_units"] > TOPK]
        assert len(full) >= 8 and all(len(b["order"][0]) == TOPK for b in full)      # a real top-k ran, not "all units"
        assert fol.stats["selections"] == len(full) == sum(1 for p, n in _blocks_of(calls) if _units_after(p) > TOPK)
        assert fol.stats["picks"] == H * cm.num_global_block
        assert cm.stats["misses"] > 0 and cm.stats["evictions"] > 0
        assert_tie_stats(fol, f"config 4, layer {i}")


def test_config4_full_size_thirty_two_layers_prefill_and_greedy_steps(monkeypatch):
    from infllm_amd.utils import GreedySearch
    dev = torch.device("cuda:0")
    layers = _watch_appends(monkeypatch, keep_tensors=False)
    model = _llama3_8b_shape(32, dev)
    T, steps = 131072, 128
    ids = torch.randint(0, VOCAB, (T,), generator=torch.Generator().manual_seed(5))
    gs = GreedySearch(model, _Tok())
    finite = []
    plain_step = gs._step

    def step(ids_, mask, past):
        logits, past = plain_step(ids_, mask, past)
        finite.append(bool(torch.isfinite(logits[:, -1].float()).all()))
        return logits, past

    gs._step = step
    text = gs.generate(input_ids=ids, max_length=steps, chunk_size=8192)[0]
    torch.cuda.synchronize()
    # greedy_search.py:52-70: the prompt without its last token in pieces of chunk_size, the last token, one token per step
    calls = [8192] * 15 + [8191] + [1] * (1 + steps)
    assert sum(calls) == T + steps and len(finite) == len(calls) and all(finite)
    assert len(text) == steps and all(0 <= t < VOCAB for t in text)
    blocks = _blocks_of(calls)
    selected = sum(min(TOPK, _units_after(p)) for p, n in blocks)
    assert len(layers) == 32 and len(gs.past_kv) == 32
    for i, rec in enumerate(layers):
        cm = rec["cm"]
        assert cm is gs.past_kv[i]
        assert rec["calls"] == calls, (i, rec["calls"][:20])
        consumed = 0
        for L, n in zip(calls, rec["units"]):
            consumed += L
            assert n == _units_after(consumed), (i, consumed, n)
        assert rec["units"][16] == 991                         # after the prompt's last token
        assert cm.length == T + steps and cm.num_global_block == _units_after(T + steps) == 992
        assert cm.stats["blocks"] == len(blocks)
        assert cm.stats["hits"] + cm.stats["misses"] == selected, (i, cm.stats, selected)
        assert cm.stats["misses"] > 0 and cm.stats["hits"] > 0
