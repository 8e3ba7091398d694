"""CPU-only checks: the C ABI library loads and exports what the header declares, the
host-side cache policy equals the oracle's model, RotaryEmbeddingESM equals the oracle."""
import os
import random
import re

import pytest
import torch

from infllm_amd import _lib
from infllm_amd.attention import ATTN_FORWRAD, ContextManager, RotaryEmbeddingESM
from infllm_amd.attention.context_manager import CachePolicy
from oracle.rope import RopeOracle
from oracle.stream import UnitCacheModel

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_library_exports_every_declared_symbol():
    header = open(os.path.join(ROOT, "include", "infllm_hip.h")).read()
    declared = set(re.findall(r"\b(infllm_[a-z_]+)\s*\(", header))
    assert declared, "no declarations found"
    lib = _lib.load()
    assert declared == set(_lib.SYMBOLS), declared ^ set(_lib.SYMBOLS)
    for name in declared:
        assert getattr(lib, name) is not None
    assert lib.infllm_version() == _lib.ABI_VERSION


def test_argument_errors_are_reported_not_raised_across_the_abi():
    lib = _lib.load()
    assert lib.infllm_ingest(None, None) < 0
    assert b"null" in lib.infllm_last_error()
    assert lib.infllm_copy_async(None, None, 4, 1, None) < 0
    assert lib.infllm_score_topk(None, 0, 0, 0, None, 0, None, None, None) < 0
    with pytest.raises(_lib.InfLLMHipError):
        _lib.check(-1, "probe")


def test_struct_layouts_match_header_sizes():
    # sizes follow from the field lists in include/infllm_hip.h under natural alignment
    import ctypes
    assert ctypes.sizeof(_lib.Page) == 32
    assert ctypes.sizeof(_lib.IngestArgs) == 3 * 8 + 9 * 8 + 4 * 4 + 2 * 8 + 8 + 8 + 4 * 8 + 8 + 3 * 8
    assert ctypes.sizeof(_lib.AttnArgs) == 8 + 24 + 16 + 16 + 48 + 24 + 8 + 16 + 8 + 8 + 8 + 16
    assert ctypes.sizeof(_lib.ScoreArgs) == 8 + 24 + 16 + 8 + 24 + 24 + 8 + 16 + 8 + 8 + 8 + 24


@pytest.mark.parametrize("strategy", ["lru", "fifo"])
def test_cache_policy_equals_oracle_model(strategy):
    rng = random.Random(5)
    pol, model = CachePolicy(6, strategy, None), UnitCacheModel(6, strategy, None)
    n_units = 3
    for step in range(300):
        n_units += rng.randint(0, 2)
        sel = sorted(rng.sample(range(n_units), min(3, n_units)))
        misses, evicted = pol.touch(sel)
        model.touch(sel)
        assert sorted(misses) == model.events[-1]["misses"]
        assert evicted == model.events[-1]["evicted"]
        assert pol.cached == model.cached
        assert set(pol.slot_of) == set(pol.cached)
        assert len(set(pol.slot_of.values())) == len(pol.slot_of)
        assert sorted(list(pol.slot_of.values()) + pol.free) == list(range(6))


def test_cache_policy_lru_s_equals_oracle_model():
    rng = random.Random(6)
    pol, model = CachePolicy(5, "lru-s", 0.9), UnitCacheModel(5, "lru-s", 0.9)
    for step in range(200):
        sel = sorted(rng.sample(range(12), 3))
        _, evicted = pol.touch(sel)
        model.touch(sel)
        assert evicted == model.events[-1]["evicted"]
        sc = [rng.random() for _ in sel]
        pol.add_scores(sel, sc)
        model.add_scores(sel, sc)
        assert pol.cached == model.cached


def test_rotary_module_matches_oracle_on_cpu():
    torch.manual_seed(0)
    mod = RotaryEmbeddingESM(16, base=1e6, distance_scale=1.0, device="cpu")
    ora = RopeOracle(16, base=1e6)
    assert torch.equal(mod.inv_freq, ora.inv_freq)
    q, k = torch.randn(1, 2, 5, 16), torch.randn(1, 1, 12, 16)
    mq, mk = mod(q, k)
    oq, ok = ora.window(q, k)
    assert torch.allclose(mq, oq, atol=1e-6) and torch.allclose(mk, ok, atol=1e-6)
    assert torch.allclose(mod.apply_rotary_pos_emb_one_angle(q, 9), ora.one_angle(q, 9), atol=1e-6)


def test_constructor_contract():
    rope = RotaryEmbeddingESM(128, device="cpu")
    assert set(ATTN_FORWRAD) >= {"inf-llm"}
    cm = ContextManager(rope, 128, 4096, 128, 32, 16, 512, None, False, 4, "lru", None, False, False, False, False)
    assert cm.length == 0 and cm.size() == 0
    with pytest.raises(AssertionError):
        ContextManager(rope, 128, 256, 128, 32, 16, 512)          # exc_block_size > n_local
    with pytest.raises(AssertionError):
        ContextManager(rope, 128, 4096, 128, 32, 16, 512, cache_strategy="mru")
    fwd = ATTN_FORWRAD["inf-llm"](n_local=4096, n_init=128, topk=16, block_size=128, max_cached_block=32,
                                  exc_block_size=512, fattn=False, repr_topk=4, type="inf-llm", path="x")
    assert callable(fwd)


def test_missing_library_fails_loudly(monkeypatch, tmp_path):
    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "LIB_PATH", str(tmp_path / "absent.so"))
    with pytest.raises(_lib.InfLLMHipError):
        _lib.load()
