"""Model-side glue on the CPU: patch_hf wiring on the installed transformers classes and the call schedule
of GreedySearch (inf_llm/utils/patch.py:33-172, greedy_search.py:35-105).  No GPU, no HIP library: the
attention type is a stand-in, or the CPU oracle."""
import copy

import pytest
import torch

from infllm_amd import attention
from infllm_amd.utils import GreedySearch, patch_hf

transformers = pytest.importorskip("transformers")


def _tiny(kind="llama", layers=2, heads=2, kv=1, hidden=256, vocab=500):
    kw = dict(hidden_size=hidden, intermediate_size=2 * hidden, num_hidden_layers=layers, num_attention_heads=heads,
              num_key_value_heads=kv, head_dim=128, vocab_size=vocab, rope_theta=500000.0)
    torch.manual_seed(0)
    if kind == "llama":
        return transformers.LlamaForCausalLM(transformers.LlamaConfig(**kw))
    if kind == "mistral":
        return transformers.MistralForCausalLM(transformers.MistralConfig(**kw))
    return transformers.Qwen2ForCausalLM(transformers.Qwen2Config(**kw))


@pytest.fixture
def counting_type():
    seen = []

    def factory(**kw):
        def forward(self, query, key_value, position_bias, use_cache, past, pq, pk, pv, po, dim_head, heads, kv_heads):
            seen.append((dim_head, heads, kv_heads, position_bias.base, past))
            out = po(pq(query))
            return (out, (past or 0) + query.size(1)) if use_cache else out
        return forward
    attention.ATTN_FORWRAD["counting"] = factory
    yield seen
    del attention.ATTN_FORWRAD["counting"]


@pytest.mark.parametrize("kind", ["llama", "mistral", "qwen2"])
def test_patch_hf_hands_each_layer_its_own_cache(kind, counting_type):
    model = patch_hf(_tiny(kind, layers=3), "counting")
    ids = torch.randint(0, 500, (1, 7))
    out = model(input_ids=ids, use_cache=True, return_dict=True)
    assert out.logits.shape == (1, 7, 500) and out.past_key_values == (7, 7, 7)
    assert [s[:4] for s in counting_type] == [(128, 2, 1, 500000.0)] * 3 and all(s[4] is None for s in counting_type)
    out = model(input_ids=ids[:, :2], use_cache=True, return_dict=True, past_key_values=out.past_key_values)
    assert out.past_key_values == (9, 9, 9) and [s[4] for s in counting_type[3:]] == [7, 7, 7]
    assert model.model.position_bias.dim == 128 and hasattr(model.model, "_old_forward")
    with pytest.raises(ValueError):
        patch_hf(torch.nn.Linear(2, 2))


def test_patch_hf_overrides_base_and_forwards_type_arguments():
    got = {}

    def factory(**kw):
        got.update(kw)
        return lambda self, q, kv, rope, use_cache, past, pq, pk, pv, po, d, h, hk: (po(pq(q)), rope)
    attention.ATTN_FORWRAD["probe"] = factory
    try:
        model = patch_hf(_tiny(), "probe", {"n_local": 64}, base=12345.0, distance_scale=2.0, topk=3)
        out = model(input_ids=torch.zeros((1, 2), dtype=torch.long), use_cache=True, return_dict=True)
        rope = out.past_key_values[0]
        assert got == {"n_local": 64, "topk": 3} and rope.base == 12345.0 and rope.distance_scale == 2.0
    finally:
        del attention.ATTN_FORWRAD["probe"]


def test_yaml_configuration_feeds_patch_hf_like_the_reference_driver(tmp_path):
    """A run configuration in the reference's layout (config/*.yaml), loaded with the defaults and command-line
    overrides of benchmark/pred.py:22-40, and its model section handed to patch_hf wholesale (pred.py:56)."""
    from infllm_amd.utils import load_config, patch_from_config
    path = tmp_path / "run.yaml"
    path.write_text("model:\n  type: probe\n  path: some/model\n  block_size: 128\n  n_init: 128\n  n_local: 4096\n"
                    "  topk: 16\n  repr_topk: 4\n  max_cached_block: 32\n  exc_block_size: 512\n  fattn: false\n"
                    "  base: 1000000\n  distance_scale: 1.0\n\nmax_len: 2147483647\nchunk_size: 8192\nconv_type: mistral-inst\n")
    conf = load_config(str(path), ["model.topk=8", "--model.score_decay=0.1", "extra.note=hello", "chunk_size=4096"])
    assert conf.model.topk == 8 and conf.model.score_decay == 0.1 and conf.extra.note == "hello" and conf.chunk_size == 4096
    assert conf.model.tokenizer_path == "some/model" and conf.truncation is None and conf.model.fattn is False
    assert conf.max_len == 2147483647 and conf["model"]["n_local"] == 4096
    got = {}

    def factory(**kw):
        got.update(kw)
        return lambda self, q, kv, rope, use_cache, past, pq, pk, pv, po, d, h, hk: (po(pq(q)), rope)
    attention.ATTN_FORWRAD["probe"] = factory
    try:
        model = patch_from_config(_tiny(), conf)
        rope = model(input_ids=torch.zeros((1, 2), dtype=torch.long), use_cache=True, return_dict=True).past_key_values[0]
    finally:
        del attention.ATTN_FORWRAD["probe"]
    # base / distance_scale go to the rotary embedding, everything else (type and paths included) to the attention type
    assert rope.base == 1000000 and rope.distance_scale == 1.0
    assert got["topk"] == 8 and got["n_local"] == 4096 and got["path"] == "some/model" and "base" not in got
    # the real attention types swallow the keys that are not theirs (inf_llm.py:5-18 ends in *args, **kwargs)
    conf.model.type = "inf-llm"
    assert callable(attention.ATTN_FORWRAD[conf.model.type](**{k: v for k, v in conf.model.items() if k not in ("base", "distance_scale")}))
    for bad in (["model.topk"], ["=3"]):
        with pytest.raises(ValueError):
            load_config(str(path), bad)
    (tmp_path / "empty.yaml").write_text("max_len: 3\n")
    with pytest.raises(ValueError):
        load_config(str(tmp_path / "empty.yaml"))


class _Tok:
    eos_token_id = 1

    def encode(self, text):
        return [int(t) for t in text.split()]

    def decode(self, ids):
        return " ".join(str(int(i)) for i in ids)


class _Recorder(torch.nn.Module):
    """A 'model' that records every call and emits a scripted token sequence."""

    def __init__(self, script, vocab=50):
        super().__init__()
        self.p = torch.nn.Parameter(torch.zeros(1))
        self.script, self.vocab, self.calls = list(script), vocab, []

    def forward(self, input_ids, attention_mask, use_cache, return_dict, past_key_values):
        self.calls.append((input_ids[0].tolist(), attention_mask.shape[1], past_key_values))
        logits = torch.zeros((1, input_ids.shape[1], self.vocab))
        past = (past_key_values or 0) + input_ids.shape[1]
        if past >= self.first_len:                      # a generation step: emit the next scripted token
            logits[0, -1, self.script[past - self.first_len]] = 1.0
        return type("Out", (), {"logits": logits, "past_key_values": past})()


def test_greedy_search_call_schedule_and_cache_reuse():
    prompt = list(range(10, 20))                        # 10 tokens
    rec = _Recorder([7, 8, 9, 1, 5])
    rec.first_len = 10
    gs = GreedySearch(rec, _Tok())
    out = gs.generate(input_ids=torch.tensor(prompt), max_length=20, chunk_size=4)
    # prefill: tokens 0..8 in pieces of 4, then the last prompt token alone; then one token per step
    assert [c[0] for c in rec.calls] == [prompt[0:4], prompt[4:8], prompt[8:9], prompt[9:10], [7], [8], [9]]
    assert [c[1] for c in rec.calls] == [4, 8, 9, 10, 11, 12, 13]            # attention_mask[:, :ed], then the full mask
    assert [c[2] for c in rec.calls] == [None, 4, 8, 9, 10, 11, 12]          # the caches are threaded through
    assert out == ["7 8 9"] and gs.past_kv == 13                              # stopped at eos (1), cache kept
    # second turn continues on the kept cache; clear() drops it
    rec.calls.clear()
    rec.first_len, rec.script = 13 + 3, [4, 1]
    assert gs.generate(text="30 31 32", max_length=5, chunk_size=None) == ["4"]
    assert [c[0] for c in rec.calls] == [[30, 31], [32], [4]] and rec.calls[0][2] == 13
    gs.clear()
    assert gs.past_kv is None


def test_greedy_search_stops_at_max_length_and_extra_end_tokens():
    rec = _Recorder([3] * 50)
    rec.first_len = 2
    gs = GreedySearch(rec, _Tok())
    assert gs.generate(input_ids=torch.tensor([[5, 6]]), max_length=4, chunk_size=8) == ["3 3 3 3"]
    assert len(rec.calls) == 1 + 1 + 4                                        # 1 prefill piece, last token, 4 steps
    gs.clear()
    rec.calls.clear()
    rec.script = [3, 9, 3]
    assert gs.generate(input_ids=torch.tensor([5, 6]), max_length=4, extra_end_token_ids=[9], chunk_size=8) == ["3"]


def test_patched_model_equals_oracle_attention_on_the_same_weights():
    """The wiring adds nothing of its own: a decoder patched with the oracle-backed type gives, for a stream inside
    the local window, the logits of the unpatched model (plain causal attention with the same RoPE base)."""
    from oracle.model_glue import oracle_inf_llm_forward
    attention.ATTN_FORWRAD["oracle-inf-llm"] = oracle_inf_llm_forward
    try:
        plain = _tiny().eval()
        patched = patch_hf(copy.deepcopy(plain), "oracle-inf-llm", n_local=64, n_init=4, topk=2, block_size=8,
                           max_cached_block=4, exc_block_size=16, repr_topk=2)
        ids = torch.randint(0, 500, (1, 40))
        with torch.no_grad():
            want = plain(input_ids=ids).logits
            a = patched(input_ids=ids[:, :25], use_cache=True, return_dict=True)
            b = patched(input_ids=ids[:, 25:], use_cache=True, return_dict=True, past_key_values=a.past_key_values)
        got = torch.cat((a.logits, b.logits), dim=1)
        assert torch.allclose(got, want, atol=2e-4), float((got - want).abs().max())
        assert all(c.length == 40 for c in b.past_key_values)
    finally:
        del attention.ATTN_FORWRAD["oracle-inf-llm"]
