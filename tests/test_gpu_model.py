"""A tiny random Llama decoder patched with the "inf-llm" attention type and driven by GreedySearch on the GPU,
against the same weights in fp32 on the CPU patched with the oracle-backed type (oracle.model_glue).

Tolerance: the GPU model runs its projections, MLP and logits in bf16 (torch's own GEMMs), the CPU copy in fp32,
so logits are compared at 6e-2 absolute for logits of unit scale, and a generated token may differ only where
the CPU model's two best logits are closer than that."""
import copy

import pytest
import torch

from oracle.model_glue import oracle_inf_llm_forward

pytestmark = pytest.mark.gpu
transformers = pytest.importorskip("transformers")

# topk covers every unit of the streams used here: the two models see slightly different activations (bf16 vs
# fp32 weights), so a real top-k could legitimately pick different units; which units are retrieved from equal
# inputs is what tests/test_gpu_stream.py pins.  Here every carved unit is attended (through the unit cache).
KNOBS = dict(n_local=128, n_init=8, topk=16, block_size=16, max_cached_block=16, exc_block_size=32, repr_topk=2, fattn=False)
LOGIT_TOL = 6e-2


def _models(head_dim=128):
    from infllm_amd import attention
    from infllm_amd.utils import patch_hf
    torch.manual_seed(1)
    cfg = transformers.LlamaConfig(hidden_size=256, intermediate_size=512, num_hidden_layers=2, num_attention_heads=256 // head_dim,
                                   num_key_value_heads=128 // head_dim, head_dim=head_dim, vocab_size=300, rope_theta=500000.0)
    base = transformers.LlamaForCausalLM(cfg).bfloat16().eval()
    attention.ATTN_FORWRAD["oracle-inf-llm"] = oracle_inf_llm_forward
    cpu = patch_hf(copy.deepcopy(base).float(), "oracle-inf-llm", dict(KNOBS))
    gpu = patch_hf(copy.deepcopy(base).cuda(), "inf-llm", dict(KNOBS))
    return gpu, cpu


class _Tok:
    eos_token_id = -1

    def decode(self, ids):
        return " ".join(str(int(i)) for i in ids)


@pytest.mark.parametrize("head_dim", [128, 64])
def test_chunked_prefill_logits_and_greedy_tokens_follow_the_cpu_model(head_dim):
    from infllm_amd.attention import ContextManager
    from infllm_amd.utils import GreedySearch
    gpu, cpu = _models(head_dim)
    ids = torch.randint(0, 300, (1, 333), generator=torch.Generator().manual_seed(2))
    with torch.inference_mode():
        past_g = past_c = None
        for st, ed in ((0, 100), (100, 101), (101, 260), (260, 333)):       # uneven calls, one single-token call
            og = gpu(input_ids=ids[:, st:ed].cuda(), use_cache=True, return_dict=True, past_key_values=past_g)
            oc = cpu(input_ids=ids[:, st:ed], use_cache=True, return_dict=True, past_key_values=past_c)
            past_g, past_c = og.past_key_values, oc.past_key_values
            err = (og.logits.float().cpu() - oc.logits).abs()
            assert float(err.max()) <= LOGIT_TOL, (st, ed, float(err.max()), float(oc.logits.std()))
    assert all(isinstance(c, ContextManager) and c.length == 333 for c in past_g)
    assert past_g[0].num_global_block == past_c[0].n_units == 12                # units were carved and attended
    assert past_g[0].stats["misses"] > 0

    gpu, cpu = _models(head_dim)
    text_g = GreedySearch(gpu, _Tok()).generate(input_ids=ids[0], max_length=8, chunk_size=64)[0].split()
    gs_c = GreedySearch(cpu, _Tok())
    text_c = gs_c.generate(input_ids=ids[0], max_length=8, chunk_size=64)[0].split()
    assert len(text_g) == len(text_c) == 8
    if text_g != text_c:                      # allowed only at a near-tie of the CPU model's logits
        first = next(i for i in range(8) if text_g[i] != text_c[i])
        cpu2 = _models(head_dim)[1]
        seq = torch.cat((ids, torch.tensor([[int(t) for t in text_c[:first]]], dtype=ids.dtype)), dim=1)
        with torch.inference_mode():
            logits = cpu2(input_ids=seq, use_cache=True, return_dict=True).logits[0, -1]
        top = logits.topk(2).values
        assert float(top[0] - top[1]) <= LOGIT_TOL, (text_g, text_c)
