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
    assert lib.infllm_layer_set_batch(None, None) < 0 and lib.infllm_call_front(None, None, None) < 0
    assert lib.infllm_layer_staged_units(None) < 0 and lib.infllm_layer_fetched_units(None) < 0
    with pytest.raises(_lib.InfLLMHipError):
        _lib.check(-1, "probe")


def test_struct_layouts_match_header_sizes():
    # sizes follow from the field lists in include/infllm_hip.h under natural alignment
    import ctypes
    assert ctypes.sizeof(_lib.Page) == 32
    assert ctypes.sizeof(_lib.IngestArgs) == 3 * 8 + 9 * 8 + 4 * 4 + 2 * 8 + 8 + 8 + 4 * 8 + 8 + 3 * 8
    assert ctypes.sizeof(_lib.AttnArgs) == 8 + 24 + 16 + 16 + 48 + 24 + 8 + 16 + 8 + 8 + 8 + 16
    assert ctypes.sizeof(_lib.ScoreArgs) == 8 + 24 + 16 + 8 + 24 + 24 + 8 + 16 + 8 + 8 + 8 + 24
    assert ctypes.sizeof(_lib.BatchDesc) == 6 * 8 + 8 + 2 * 4


@pytest.mark.parametrize("strategy", ["lru", "fifo"])
def test_cache_policy_equals_oracle_model(strategy):
    rng = random.Random(5)
    pol, model = CachePolicy(6, strategy, None), UnitCacheModel(6, strategy, None)
    n_units = 3
    for step in range(300):
        n_units += rng.randint(0, 2)
        sel = rng.sample(range(n_units), min(3, n_units))           # an ordered list, as torch.topk returns it
        misses, evicted = pol.touch(sel)
        model.touch(sel)
        assert sorted(misses) == model.events[-1]["misses"]
        assert misses == [u for u in sel if u in misses]              # misses are reported in selection order
        assert evicted == model.events[-1]["evicted"]
        assert pol.cached == model.cached
        assert set(pol.slot_of) == set(pol.cached)
        assert len(set(pol.slot_of.values())) == len(pol.slot_of)
        assert sorted(list(pol.slot_of.values()) + pol.free) == list(range(6))


@pytest.mark.parametrize("strategy", ["lru", "fifo"])
def test_trying_a_selection_out_on_a_copy_leaves_the_policy_as_the_oracle_model_has_it(strategy):
    """The protocol of the fetch ahead of the selection, on the host alone: a guessed selection is applied to a clone
    (infllm_cache_clone / _copy); when the real selection equals the guess the clone becomes the state, otherwise the
    real selection is applied to the untouched state with the guess's slots as wishes (infllm_cache_touch_hinted).
    Either way misses, evictions and residency follow the oracle's model, every unit sits in a slot of its own, a
    wish is granted exactly when the slot is free after the evictions, and a unit whose wish was granted keeps the
    slot the guess gave it."""
    import ctypes
    lib = _lib.load()
    rng = random.Random(11)
    cap, k = 7, 3
    pol, model = CachePolicy(cap, strategy, None), UnitCacheModel(cap, strategy, None)
    shadow = lib.infllm_cache_clone(pol.handle)
    assert shadow
    I = ctypes.c_int32
    n_units, confirmed, refuted, granted_total = 4, 0, 0, 0
    try:
        for step in range(400):
            n_units += rng.randint(0, 2)
            guess = rng.sample(range(n_units), k)
            real = guess
            if rng.random() < 0.4:                       # as in the stream: a fresh unit displaces one of the guess
                others = [u for u in range(n_units) if u not in guess]
                real = rng.sample(guess, k - 1)
                real.insert(rng.randrange(k), rng.choice(others))
            before = dict(pol.slot_of)
            assert lib.infllm_cache_copy(shadow, pol.handle) == 0
            g_slots, g_mu, g_ms, g_ev, g_nev = (I * k)(), (I * k)(), (I * k)(), (I * cap)(), I(0)
            g_miss = lib.infllm_cache_touch(shadow, (I * k)(*guess), k, g_slots, g_mu, g_ms, g_ev, ctypes.byref(g_nev))
            assert g_miss >= 0 and pol.slot_of == before                  # the guess has not touched the real state
            for u in before:
                assert lib.infllm_cache_slot_of(pol.handle, u) == before[u]
            assert lib.infllm_cache_slot_of(pol.handle, n_units + 5) == -1
            model.touch(real)
            want = model.events[-1]
            if real == guess:
                confirmed += 1
                assert lib.infllm_cache_copy(pol.handle, shadow) == 0
                assert sorted(g_mu[:g_miss]) == want["misses"] and list(g_ev[:g_nev.value]) == want["evicted"]
            else:
                refuted += 1
                slots, mu, ms, ev, nev = (I * k)(), (I * k)(), (I * k)(), (I * cap)(), I(0)
                n_miss = lib.infllm_cache_touch_hinted(pol.handle, (I * k)(*real), k, slots, mu, ms, ev, ctypes.byref(nev),
                                                       g_mu, g_ms, g_miss)
                assert sorted(mu[:n_miss]) == want["misses"] and list(ev[:nev.value]) == want["evicted"]
                hint = dict(zip(g_mu[:g_miss], g_ms[:g_miss]))
                freed = {before[u] for u in want["evicted"]}
                free_then = (set(range(cap)) - set(before.values())) | freed
                for u, sl in zip(mu[:n_miss], ms[:n_miss]):
                    if u in hint and hint[u] in free_then:
                        assert sl == hint[u]
                        granted_total += 1
            assert pol.cached == model.cached
            assert len(set(pol.slot_of.values())) == len(pol.slot_of) and set(pol.slot_of) == set(pol.cached)
    finally:
        lib.infllm_cache_destroy(shadow)
    assert confirmed > 50 and refuted > 50 and granted_total > 20
    other = CachePolicy(cap + 1, strategy, None)
    assert lib.infllm_cache_copy(other.handle, pol.handle) != 0          # different capacity: refused


def test_units_missed_in_one_block_are_inserted_in_selection_order():
    """context_manager.py:495-515 walks the torch.topk list (descending score), so the units a block loads together
    enter the dict in that order, and the order decides which of them leaves first once their stamps tie
    (:253-265, a stable sort).  Capacity 4, selections [5,2], [7,8], [9,7]: the third block must evict 5, the unit
    inserted first; with the ids sorted it would be 2."""
    pol, model = CachePolicy(4, "lru", None), UnitCacheModel(4, "lru", None)
    for sel, want in (([5, 2], []), ([7, 8], []), ([9, 7], [5])):
        misses, evicted = pol.touch(sel)
        model.touch(sel)
        assert evicted == want == model.events[-1]["evicted"]
    assert list(pol.cached) == list(model.cached) == [2, 7, 8, 9]
    # the reference's dict in plain Python, for the same three blocks
    cached, clock = {}, 0
    for sel in ([5, 2], [7, 8], [9, 7]):
        surplus = len(cached) - 4 + sum(b not in cached for b in sel)
        for unit, _ in sorted(cached.items(), key=lambda kv: kv[1]):
            if surplus <= 0:
                break
            if unit not in sel:
                del cached[unit]
                surplus -= 1
        clock += 1
        for b in sel:
            cached[b] = clock
    assert list(cached) == [2, 7, 8, 9]


def test_cache_policy_lru_s_equals_oracle_model():
    rng = random.Random(6)
    pol, model = CachePolicy(5, "lru-s", 0.9), UnitCacheModel(5, "lru-s", 0.9)
    for step in range(200):
        sel = rng.sample(range(12), 3)
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


def test_bench_refuses_more_than_one_gpu_with_a_message():
    """bench.py --gpus N with N above 1 exits with a message that says why (no GPU is touched on that path)."""
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    p = subprocess.run([sys.executable, os.path.join(root, "bench.py"), "--gpus", "2"], capture_output=True, text=True, timeout=300)
    assert p.returncode != 0 and "ONE GPU" in p.stderr and p.stdout.strip() == ""
