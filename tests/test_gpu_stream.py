"""End-to-end parity of the streaming path on the GPU against the CPU oracle.

The GPU ContextManager and oracle.stream.StreamOracle consume the same
bf16-rounded stream.  Discrete choices (retrieved unit sets, representative
keys) must be identical except where the oracle's own fp32 scores of the
candidates that differ lie within 1e-3 relative of the selection boundary; in
that case the oracle adopts the GPU's choice (so that the two trajectories stay
comparable) and the event is counted.  Outputs must agree within max-abs 2e-2 /
mean-abs 2e-3.
"""
import pytest
import torch

from oracle.rope import RopeOracle
from oracle.stream import StreamOracle

pytestmark = pytest.mark.gpu

MAX_ABS, MEAN_ABS, TIE_REL = 2e-2, 2e-3, 1e-3
D = 128


def _stream(T, H, Hkv, seed, B=1, mixture=True):
    """q, v ~ N(0,1); keys from a 64-component Gaussian mixture (std 0.3 around N(0,1) means)."""
    g = torch.Generator().manual_seed(seed)
    q = torch.randn(B, H, T, D, generator=g)
    v = torch.randn(B, Hkv, T, D, generator=g)
    if mixture:
        means = torch.randn(Hkv, 64, D, generator=g)
        comp = torch.randint(0, 64, (B, Hkv, T), generator=g)
        k = torch.stack([means[h][comp[:, h]] for h in range(Hkv)], dim=1) + 0.3 * torch.randn(B, Hkv, T, D, generator=g)
    else:
        k = torch.randn(B, Hkv, T, D, generator=g)
    return q.bfloat16(), k.bfloat16(), v.bfloat16()


def _run_gpu(q, k, v, calls, base, **kw):
    from infllm_amd.attention import ContextManager, RotaryEmbeddingESM
    rope = RotaryEmbeddingESM(D, base=base, device="cuda")
    cm = ContextManager(rope, kw["n_init"], kw["n_local"], kw["block_size"], kw["max_cached_block"], kw["topk"],
                        kw["exc_block_size"], kw.get("score_decay"), False, kw.get("repr_topk", 1),
                        kw.get("cache_strategy", "lru"), kw.get("chunk_topk_calc"), kw.get("async_global_stream", False), False, False,
                        kw.get("perhead", False))
    cm.record_trace = True
    qd, kd, vd = q.cuda(), k.cuda(), v.cuda()
    outs, pos = [], 0
    for L in calls:
        sl = slice(pos, pos + L)
        outs.append(cm.append(qd[:, :, sl], kd[:, :, sl], vd[:, :, sl], qd[:, :, sl], kd[:, :, sl], vd[:, :, sl]))
        pos += L
    torch.cuda.synchronize()
    return torch.cat(outs, dim=2).cpu(), cm


class Follower:
    """Oracle hooks that adopt the GPU's choices when the tie rule allows it."""

    def __init__(self, cm, topk, repr_topk):
        self.blocks = cm.trace_blocks
        self.repr = cm.trace_repr_indices()
        self.topk, self.repr_topk = topk, repr_topk
        self.tie_topk = self.tie_repr = 0
        self.violations = []

    def topk_hook(self, block, row, scores):
        gpu = set(self.blocks[block]["selected"][row])
        mine = set(scores.topk(self.topk).indices.tolist())
        if gpu == mine:
            return None
        kth = float(scores.topk(self.topk).values[-1])
        bad = [i for i in gpu ^ mine if abs(float(scores[i]) - kth) > TIE_REL * abs(kth)]
        if bad:
            self.violations.append(("topk", block, row, bad))
        self.tie_topk += 1
        return sorted(gpu)

    def repr_hook(self, unit, row, score):
        gpu = self.repr[unit][row].long()                      # [H, r]
        mine = score.topk(self.repr_topk, dim=-1)
        for h in range(score.shape[0]):
            a, b = set(gpu[h].tolist()), set(mine.indices[h].tolist())
            if a != b:
                rth = float(mine.values[h, -1])
                bad = [i for i in a ^ b if abs(float(score[h, i]) - rth) > TIE_REL * abs(rth)]
                if bad:
                    self.violations.append(("repr", unit, row, h, bad))
                self.tie_repr += 1
        return gpu


def _compare(T, calls, H, Hkv, base, seed, B=1, **kw):
    q, k, v = _stream(T, H, Hkv, seed, B=B)
    got, cm = _run_gpu(q, k, v, calls, base, **kw)
    fol = Follower(cm, kw["topk"], kw.get("repr_topk", 1))
    ora = StreamOracle(RopeOracle(D, base=base), kw["n_init"], kw["n_local"], kw["block_size"], kw["max_cached_block"],
                       kw["topk"], kw["exc_block_size"], repr_topk=kw.get("repr_topk", 1), perhead=kw.get("perhead", False),
                       topk_hook=fol.topk_hook, repr_hook=fol.repr_hook, cache_strategy=kw.get("cache_strategy", "lru"),
                       score_decay=kw.get("score_decay"), chunk_topk_calc=kw.get("chunk_topk_calc"))
    outs, pos = [], 0
    for L in calls:
        sl = slice(pos, pos + L)
        outs.append(ora.append(q[:, :, sl].float(), k[:, :, sl].float(), v[:, :, sl].float()))
        pos += L
    want = torch.cat(outs, dim=2)
    assert not fol.violations, fol.violations[:5]
    assert [b["selected"] for b in cm.trace_blocks] == [b["selected"] for b in ora.block_trace]
    assert cm.num_global_block == ora.n_units and cm.length == ora.length == T
    err = (got.float() - want).abs()
    assert float(err.max()) <= MAX_ABS and float(err.mean()) <= MEAN_ABS, (float(err.max()), float(err.mean()))
    # the cache model saw the same selections, so residency events must match too
    if not kw.get("perhead", False):
        hits = sum(len(e["selected"]) - len(e["misses"]) for c in ora.cache for e in c.events)
        assert cm.stats["hits"] == hits
    return cm, ora, fol


SMALL = dict(n_init=16, n_local=256, block_size=32, max_cached_block=8, topk=4, exc_block_size=64, repr_topk=2)


@pytest.mark.parametrize("calls", [[1500], [64] * 20 + [100, 17, 3], [1] * 40 + [700] + [1] * 30])
def test_small_geometry_follows_oracle(calls):
    cm, ora, fol = _compare(sum(calls), calls, H=8, Hkv=2, base=1e4, seed=len(calls), **SMALL)
    assert cm.num_global_block > SMALL["topk"]            # retrieval was exercised


def test_score_decay_policy_follows_oracle():
    """cache_strategy lru-s: evictions are decided by the decayed attention mass each cached unit received
    (context_manager.py:454-470), which the device computes and the host reads back once per block."""
    kw = dict(SMALL, cache_strategy="lru-s", score_decay=0.1, max_cached_block=6)
    cm, ora, _ = _compare(1500, [700, 1, 1, 798], H=8, Hkv=2, base=1e4, seed=31, B=2, **kw)
    assert cm.stats["evictions"] > 20
    for u in range(2):
        gpu_events = [sorted(e) for e in cm.policy[u].evicted_log]
        assert gpu_events == [sorted(e["evicted"]) for e in ora.cache[u].events]
        assert list(cm.policy[u].cached) == list(ora.cache[u].cached)      # same residents, same dict order
    # unit masses: every block's mass is a share of the H * n probabilities of that block
    assert 0.0 < float(cm.mass_host.sum()) <= 2 * 8 * 64 + 1e-3


@pytest.mark.parametrize("chunk", [64, 192, 4096])
def test_chunked_retrieval_follows_oracle(chunk):
    kw = dict(SMALL, chunk_topk_calc=chunk)
    cm, ora, _ = _compare(1334, [1000, 1, 333], H=8, Hkv=2, base=1e4, seed=33, B=2, **kw)
    assert cm.num_global_block > SMALL["topk"]


def test_unaligned_geometry_and_batch():
    kw = dict(n_init=5, n_local=130, block_size=24, max_cached_block=3, topk=3, exc_block_size=50, repr_topk=3)
    _compare(700, [333, 367], H=6, Hkv=3, base=1e4, seed=7, B=2, **kw)


def test_edge_knobs_and_empty_calls():
    """No attention sinks, an execution block as long as the local window, a cache exactly as large as the
    selection, one representative key per unit; calls of 1 and of 0 tokens in between."""
    kw = dict(n_init=0, n_local=64, block_size=32, max_cached_block=2, topk=2, exc_block_size=64, repr_topk=1)
    calls = [1, 63, 64, 300, 72]
    cm, ora, _ = _compare(sum(calls), calls, H=4, Hkv=2, base=1e4, seed=21, **kw)
    assert cm.init_len == 0 and cm.num_global_block == (sum(calls) - 64) // 32 and cm.stats["misses"] > 0
    # an empty call changes nothing and returns an empty result
    q, k, v = _stream(8, 4, 2, 22)
    qd, kd, vd = q.cuda(), k.cuda(), v.cuda()
    before = (cm.length, cm.num_global_block, cm.cursor)
    out = cm.append(qd[:, :, :0], kd[:, :, :0], vd[:, :, :0], qd[:, :, :0], kd[:, :, :0], vd[:, :, :0])
    assert tuple(out.shape) == (1, 4, 0, D) and (cm.length, cm.num_global_block, cm.cursor) == before


def test_many_batch_rows_take_the_host_built_page_table():
    """More than 64 selected (row, unit) pairs per block: the page table no longer fits a kernel argument and
    is staged through pinned memory instead."""
    # repr_topk = block_size: the representative is the plain mean of the unit's keys, so this test exercises the
    # page-table path without depending on near-ties among 16 noisy token scores
    kw = dict(n_init=8, n_local=128, block_size=16, max_cached_block=16, topk=16, exc_block_size=32, repr_topk=16)
    cm, ora, _ = _compare(600, [300, 300], H=4, Hkv=2, base=1e4, seed=18, B=5, **kw)
    assert cm.num_global_block > kw["topk"] and cm.num_units * kw["topk"] > 64


def test_no_gqa_and_perhead():
    kw = dict(SMALL, perhead=True)
    _compare(800, [800], H=2, Hkv=1, base=1e4, seed=8, **kw)
    _compare(800, [800], H=2, Hkv=2, base=1e4, seed=9, **SMALL)


def test_reference_geometry_16k():
    """Mistral-7B geometry and the reference's default knobs (config/mistral-inf-llm.yaml)."""
    kw = dict(n_init=128, n_local=4096, block_size=128, max_cached_block=32, topk=16, exc_block_size=512, repr_topk=4)
    T = 8192 + 1024
    cm, ora, fol = _compare(T, [8192, 1024], H=32, Hkv=8, base=1e6, seed=11, **kw)
    assert cm.num_global_block == (T - 128 - 4096) // 128 > 16


def test_call_splitting_cache_size_and_side_stream_do_not_change_results():
    T = 1280
    q, k, v = _stream(T, 8, 2, 12)
    ref, cm0 = _run_gpu(q, k, v, [T], 1e4, **SMALL)
    split, _ = _run_gpu(q, k, v, [640, 640], 1e4, **SMALL)
    assert torch.equal(ref, split)
    tight, cm1 = _run_gpu(q, k, v, [T], 1e4, **dict(SMALL, max_cached_block=4))
    assert torch.equal(ref, tight) and cm1.stats["misses"] > cm0.stats["misses"]
    side, cm2 = _run_gpu(q, k, v, [T], 1e4, **dict(SMALL, max_cached_block=4, async_global_stream=True))
    assert torch.equal(ref, side) and cm2.stats == cm1.stats
    fifo, _ = _run_gpu(q, k, v, [T], 1e4, **dict(SMALL, cache_strategy="fifo"))
    assert torch.equal(ref, fifo)


def test_carved_units_reach_the_host_by_either_copy_path(monkeypatch):
    """New units go to their pinned home through the DMA engine, or (INFLLM_NO_DMA_ENGINE=1) by a stream-ordered
    hipMemcpyAsync: same bytes on the host, same outputs (the tight cache makes later blocks fetch them back)."""
    T = 1280
    q, k, v = _stream(T, 8, 2, 14)
    kw = dict(SMALL, max_cached_block=4, async_global_stream=True)
    runs = [_run_gpu(q, k, v, [640, 500, 140], 1e4, **kw)]
    monkeypatch.setenv("INFLLM_NO_DMA_ENGINE", "1")
    runs.append(_run_gpu(q, k, v, [640, 500, 140], 1e4, **kw))
    assert torch.equal(runs[0][0], runs[1][0]) and runs[0][1].stats == runs[1][1].stats
    bs, n_init = SMALL["block_size"], SMALL["n_init"]
    for _, cm in runs:
        assert cm.num_global_block == (T - n_init - SMALL["n_local"]) // bs
        for u in range(cm.num_global_block):
            lo, hu = n_init + u * bs, cm.host_unit(u)
            assert torch.equal(hu[0, 0], k[0, :, lo:lo + bs]) and torch.equal(hu[0, 1], v[0, :, lo:lo + bs]), u


def test_fetch_ahead_of_the_selection_changes_nothing(monkeypatch):
    """The next block's misses are fetched from the candidates chosen before the block's own units are carved
    (infllm_block_prefetch).  Whether the guess is confirmed or not, outputs, hit / miss / eviction counts, the
    eviction sequence and the final residency are those of the run without it - with the units moved by the DMA
    engines and by the fetch kernel (INFLLM_NO_DMA_FETCH=1), for lru and fifo, with a tight and a roomy cache."""
    from infllm_amd.attention import ContextManager
    T = 2600
    q, k, v = _stream(T, 8, 2, 21, B=2)
    seen_confirmed = seen_refuted = 0
    for extra in (dict(max_cached_block=5), dict(max_cached_block=12), dict(max_cached_block=6, cache_strategy="fifo")):
        kw = dict(SMALL, async_global_stream=True, **extra)
        monkeypatch.setattr(ContextManager, "fetch_ahead", False)
        plain, cm0 = _run_gpu(q, k, v, [1300, 1300], 1e4, **kw)
        assert cm0.prefetch_stats() == (0, 0) and cm0.stats["misses"] > 0
        monkeypatch.setattr(ContextManager, "fetch_ahead", True)
        monkeypatch.setenv("INFLLM_FETCH_AHEAD_ALWAYS", "1")       # by default only the engines fetch ahead
        for no_dma in ("0", "1"):
            monkeypatch.setenv("INFLLM_NO_DMA_FETCH", no_dma)
            ahead, cm1 = _run_gpu(q, k, v, [1300, 1300], 1e4, **kw)
            issued, confirmed = cm1.prefetch_stats()
            assert issued > 0 and 0 <= confirmed <= issued
            seen_confirmed += confirmed
            seen_refuted += issued - confirmed
            assert torch.equal(plain, ahead) and cm0.stats == cm1.stats
            for u in range(2):
                assert cm0.policy[u].evicted_log == cm1.policy[u].evicted_log
                assert cm0.policy[u].cached == cm1.policy[u].cached            # which slot a unit sits in may differ
                assert sorted(cm1.policy[u].slot_of.values()) == sorted(set(cm1.policy[u].slot_of.values()))
        monkeypatch.delenv("INFLLM_NO_DMA_FETCH")
        monkeypatch.delenv("INFLLM_FETCH_AHEAD_ALWAYS")
    assert seen_confirmed > 0 and seen_refuted > 0          # both ways of settling a guess were exercised


def test_stage_timers_sample_the_launches_they_are_asked_for():
    """infllm_layer_timing / infllm_layer_read_timing (what bench.py's roofline figure is made of): every stride-th
    launch of the local stage, of the global stage and of the stream's wait for the fetch is bracketed by events; the
    records carry the launch's sizes and a positive duration, and timing changes no result."""
    from infllm_amd.attention import ContextManager, RotaryEmbeddingESM
    T = 1600
    q, k, v = _stream(T, 8, 2, 23)
    kw = dict(SMALL, max_cached_block=5, async_global_stream=True)
    plain, _ = _run_gpu(q, k, v, [T], 1e4, **kw)
    rope = RotaryEmbeddingESM(D, base=1e4, device="cuda")
    cm = ContextManager(rope, kw["n_init"], kw["n_local"], kw["block_size"], kw["max_cached_block"], kw["topk"],
                        kw["exc_block_size"], None, False, kw["repr_topk"], "lru", None, True, False, False, False)
    cm.enable_timing(64, 2)
    qd, kd, vd = q.cuda(), k.cuda(), v.cuda()
    out = cm.append(qd, kd, vd, qd, kd, vd)
    torch.cuda.synchronize()
    assert torch.equal(out.cpu(), plain)
    n_blocks = T // kw["exc_block_size"]
    local, glob, wait = cm.read_timing(0), cm.read_timing(1), cm.read_timing(2)
    assert len(local) == (n_blocks + 1) // 2                       # every second launch of n_blocks
    assert 0 < len(glob) <= len(local) and 0 < len(wait) <= len(glob)
    for ms, nq, nk in local + glob + wait:
        assert 0.0 < ms < 50.0 and nq == kw["exc_block_size"]
    assert max(nk for _, _, nk in local) == kw["n_local"] + kw["exc_block_size"]
    import ctypes
    from infllm_amd._lib import InfLLMHipError, check
    with pytest.raises(InfLLMHipError):                            # there is no fourth timer
        check(cm._lib.infllm_layer_read_timing(cm._layer, 3, (ctypes.c_float * 4)(), None, None, 4), "infllm_layer_read_timing")


def test_selection_in_separate_steps_equals_the_fused_call(monkeypatch):
    """infllm_layer_wait_topk + infllm_cache_touch + infllm_block_fetch, driven from the host, against
    infllm_block_select: same outputs, same residency events, for every policy."""
    from infllm_amd.attention import ContextManager
    T = 1400
    q, k, v = _stream(T, 8, 2, 15, B=2)
    for extra in (dict(), dict(cache_strategy="fifo"), dict(cache_strategy="lru-s", score_decay=0.5)):
        kw = dict(SMALL, max_cached_block=5, async_global_stream=True, **extra)
        monkeypatch.setattr(ContextManager, "select_in_steps", False)
        fused, cm0 = _run_gpu(q, k, v, [700, 700], 1e4, **kw)
        monkeypatch.setattr(ContextManager, "select_in_steps", True)
        steps, cm1 = _run_gpu(q, k, v, [700, 700], 1e4, **kw)
        assert torch.equal(fused, steps) and cm0.stats == cm1.stats and cm0.stats["misses"] > 0
        for u in range(2):
            assert cm0.policy[u].evicted_log == cm1.policy[u].evicted_log
            assert cm0.policy[u].cached == cm1.policy[u].cached
            # the slots themselves may differ: the fused call fetches ahead of the selection and keeps what it moved
            assert set(cm0.policy[u].slot_of) == set(cm1.policy[u].slot_of)
            assert len(set(cm0.policy[u].slot_of.values())) == len(cm0.policy[u].slot_of)


def test_state_export_and_injection_resume_the_stream_exactly():
    from infllm_amd.attention import ContextManager, RotaryEmbeddingESM
    T0, T1 = 900, 333
    q, k, v = _stream(T0 + T1, 8, 2, 13)
    full, cm1 = _run_gpu(q, k, v, [T0, T1], 1e4, **SMALL)
    _, cm_a = _run_gpu(q[:, :, :T0], k[:, :, :T0], v[:, :, :T0], [T0], 1e4, **SMALL)
    state = cm_a.export_state()
    assert state["n_units"] == (T0 - SMALL["n_init"] - SMALL["n_local"]) // SMALL["block_size"]
    assert torch.equal(state["init_k"].cpu(), k[:, :, :SMALL["n_init"]])
    assert torch.equal(state["tail_k"].cpu(), k[:, :, T0 - state["tail_k"].shape[2]:T0])
    u3 = state["units"][3]                                    # unit 3 = tokens [n_init + 3*bs, n_init + 4*bs)
    lo = SMALL["n_init"] + 3 * SMALL["block_size"]
    assert torch.equal(u3[0, 0], k[0, :, lo:lo + SMALL["block_size"]]) and torch.equal(u3[0, 1], v[0, :, lo:lo + SMALL["block_size"]])
    rope = RotaryEmbeddingESM(D, base=1e4, device="cuda")
    cm_b = ContextManager(rope, SMALL["n_init"], SMALL["n_local"], SMALL["block_size"], SMALL["max_cached_block"],
                          SMALL["topk"], SMALL["exc_block_size"], None, False, SMALL["repr_topk"]).load_state(state)
    assert cm_b.length == T0 and cm_b.num_global_block == state["n_units"]
    sl = slice(T0, T0 + T1)
    qd, kd, vd = q[:, :, sl].cuda(), k[:, :, sl].cuda(), v[:, :, sl].cuda()
    resumed = cm_b.append(qd, kd, vd, qd, kd, vd).cpu()
    assert torch.equal(resumed, full[:, :, sl])
    assert cm_b.length == T0 + T1 == cm1.length and cm_b.num_global_block == cm1.num_global_block


def test_full_size_stream_is_the_same_with_and_without_the_fetch_ahead(monkeypatch):
    """BASELINE config 2 at full size (131,072 tokens, Mistral geometry, mixture keys, 32 slots for 16 selected units of
    512 KiB each): the stream with the fetch ahead of the selection (DMA engines, about four of five guesses confirmed,
    the others repaired) against the stream without it - outputs bit for bit, hit / miss / eviction counts, the eviction
    sequence, the final residency, and the units' pinned host copies against the input."""
    from infllm_amd.attention import ContextManager, RotaryEmbeddingESM
    H, Hkv, T, exc, n_local, n_init, bs, topk = 32, 8, 131072, 512, 4096, 128, 128, 16
    q, k, v = _stream(T, H, Hkv, seed=101)
    qd, kd, vd = q.cuda(), k.cuda(), v.cuda()
    monkeypatch.delenv("INFLLM_NO_DMA_FETCH", raising=False)      # the engines where the process can use them ...
    monkeypatch.setenv("INFLLM_FETCH_AHEAD_ALWAYS", "1")          # ... and guesses also where it cannot

    def run(ahead):
        monkeypatch.setattr(ContextManager, "fetch_ahead", ahead)
        rope = RotaryEmbeddingESM(D, base=1e6, device="cuda")
        cm = ContextManager(rope, n_init, n_local, bs, 32, topk, exc, None, False, 4, "lru", None, True)
        outs = []
        for i, st in enumerate(range(0, T, 8192)):
            sl = slice(st, st + 8192)
            if i == 1:
                cm.policy[0].evicted_log = []
            outs.append(cm.append(qd[:, :, sl], kd[:, :, sl], vd[:, :, sl], qd[:, :, sl], kd[:, :, sl], vd[:, :, sl]).cpu())
        torch.cuda.synchronize()
        return torch.cat(outs, dim=2), cm

    plain, cm0 = run(False)
    ahead, cm1 = run(True)
    issued, confirmed = cm1.prefetch_stats()
    assert cm0.prefetch_stats() == (0, 0) and issued > 200 and issued // 2 < confirmed < issued
    assert torch.equal(plain, ahead)
    assert cm0.stats == cm1.stats and cm0.stats["misses"] > 3000
    assert cm0.policy[0].evicted_log == cm1.policy[0].evicted_log and cm0.policy[0].cached == cm1.policy[0].cached
    assert cm1.num_global_block == (T - n_init - n_local) // bs
    for u in range(0, cm1.num_global_block, 41):
        lo, hu = n_init + u * bs, cm1.host_unit(u)
        assert torch.equal(hu[0, 0], k[0, :, lo:lo + bs]) and torch.equal(hu[0, 1], v[0, :, lo:lo + bs]), u


def test_full_size_stream_one_block_against_the_oracle_from_exported_state():
    """BASELINE config 2 at full size (131,072 tokens, Mistral geometry, mixture keys).  The whole stream is too long
    for the CPU oracle, so: closed forms for the state, and ONE execution block (the last) recomputed on the CPU
    in fp32 from the state exported just before it - its retrieval set by brute force over all 990 representatives,
    its output through oracle.multistage with window-relative RoPE (small angles, as the reference forms them)."""
    from infllm_amd.attention import ContextManager, RotaryEmbeddingESM
    from oracle.multistage import MultiStageOracle
    H, Hkv, T, exc, n_local, n_init, bs, topk = 32, 8, 131072, 512, 4096, 128, 128, 16
    base = 1e6
    q, k, v = _stream(T, H, Hkv, seed=100)
    rope = RotaryEmbeddingESM(D, base=base, device="cuda")
    cm = ContextManager(rope, n_init, n_local, bs, 32, topk, exc, None, False, 4, "lru", None, True)
    qd, kd, vd = q.cuda(), k.cuda(), v.cuda()
    T0 = T - exc
    for st in range(0, T0, 8192):
        sl = slice(st, min(st + 8192, T0))
        cm.append(qd[:, :, sl], kd[:, :, sl], vd[:, :, sl], qd[:, :, sl], kd[:, :, sl], vd[:, :, sl])
    state = cm.export_state()
    n_units = (T0 - n_init - n_local) // bs
    assert state["n_units"] == n_units == cm.num_global_block and state["init_len"] == n_init
    n_tail = state["tail_k"].shape[2]
    assert n_tail == T0 - n_init - n_units * bs and n_local <= n_tail < n_local + bs
    assert torch.equal(state["tail_k"].cpu(), k[:, :, T0 - n_tail:T0])
    cm.record_trace = True
    sl = slice(T0, T)
    got = cm.append(qd[:, :, sl], kd[:, :, sl], vd[:, :, sl], qd[:, :, sl], kd[:, :, sl], vd[:, :, sl]).cpu()
    chosen = cm.trace_blocks[-1]["selected"][0]
    assert cm.length == T and cm.num_global_block == (T - n_init - n_local) // bs == 991

    ora_rope = RopeOracle(D, base=base)
    qb, kb, vb = q[:, :, sl].float(), k[:, :, sl].float(), v[:, :, sl].float()
    gq = ora_rope.one_angle(qb, n_local)
    # retrieval: top-16 of sum_h mean-query_h . representative_h over every unit (context_manager.py:366-383)
    scores = state["reps"][0].float().cpu().double() @ gq[0].mean(dim=1).reshape(-1).double()
    want = set(scores.topk(topk).indices.tolist())
    kth = float(scores.topk(topk).values[-1])
    assert all(abs(float(scores[i]) - kth) <= TIE_REL * abs(kth) for i in set(chosen) ^ want), (sorted(chosen), sorted(want))
    # attention of the block: local window (relative RoPE) + [chosen units | init | overflow remainder] (un-rotated)
    tail_k, tail_v = state["tail_k"].float().cpu(), state["tail_v"].float().cpu()
    all_k, all_v = torch.cat((tail_k, kb), dim=2), torch.cat((tail_v, vb), dim=2)
    win_k, win_v = all_k[:, :, -(n_local + exc):], all_v[:, :, -(n_local + exc):]
    q_rot, k_rot = ora_rope.window(qb, win_k)
    attn = MultiStageOracle(qb.shape)
    attn.append(q_rot, k_rot, win_v, sliding_window=n_local)
    overflow = max(n_tail + exc - n_local, 0)
    units = state["units"]
    glob_k = torch.cat([units[u][:, 0].float().cpu() for u in sorted(chosen)] + [state["init_k"].float().cpu(), tail_k[:, :, :overflow]], dim=2)
    glob_v = torch.cat([units[u][:, 1].float().cpu() for u in sorted(chosen)] + [state["init_v"].float().cpu(), tail_v[:, :, :overflow]], dim=2)
    assert glob_k.shape[2] == topk * bs + n_init + overflow
    attn.append(gq, glob_k, glob_v, end=True, sliding_window=(n_local + glob_k.shape[2], n_local), complement_sliding_window=True)
    want_out, _ = attn.get_result()
    err = (got.float() - want_out).abs()
    assert float(err.max()) <= MAX_ABS and float(err.mean()) <= MEAN_ABS, (float(err.max()), float(err.mean()))


def test_decode_steps_follow_oracle():
    """Single-token appends over a prepared memory (the decode shape): retrieval, fetch and attention per step."""
    calls = [1200] + [1] * 48
    cm, ora, fol = _compare(sum(calls), calls, H=8, Hkv=2, base=1e4, seed=21, **SMALL)
    assert cm.stats["blocks"] == len(ora.block_trace)


def test_attention_type_forward_contract():
    """ATTN_FORWRAD['inf-llm'] closure: projections in, (output, ContextManager) out (inf_llm.py:20-77)."""
    from infllm_amd.attention import ATTN_FORWRAD, ContextManager, RotaryEmbeddingESM
    H, Hkv, hidden, L = 4, 2, 64, 96
    torch.manual_seed(0)
    mk = lambda o: torch.nn.Linear(hidden, o, bias=False).cuda().bfloat16()
    pq, pk, pv, po = mk(H * D), mk(Hkv * D), mk(Hkv * D), torch.nn.Linear(H * D, hidden, bias=False).cuda().bfloat16()
    fwd = ATTN_FORWRAD["inf-llm"](**dict(SMALL, fattn=False, type="inf-llm"))
    rope = RotaryEmbeddingESM(D, base=1e4, device="cuda")
    x = torch.randn(1, L, hidden, device="cuda").bfloat16()
    with torch.no_grad():
        o, cm = fwd(None, x, x, rope, True, None, pq, pk, pv, po, D, H, Hkv)
        o2, cm2 = fwd(None, x[:, :1], x[:, :1], rope, True, cm, pq, pk, pv, po, D, H, Hkv)
    assert isinstance(cm, ContextManager) and cm2 is cm and cm.length == L + 1 == cm.size()
    assert o.shape == (1, L, hidden) and o2.shape == (1, 1, hidden) and torch.isfinite(o.float()).all()
    # inside the window the path is plain causal attention with standard RoPE
    q = pq(x).view(1, L, H, D).permute(0, 2, 1, 3).float().cpu()
    k = pk(x).view(1, L, Hkv, D).permute(0, 2, 1, 3).float().cpu()
    v = pv(x).view(1, L, Hkv, D).permute(0, 2, 1, 3).float().cpu()
    ro = RopeOracle(D, base=1e4)
    want = torch.nn.functional.scaled_dot_product_attention(
        ro.rotate(q, range(L)), ro.rotate(k, range(L)).repeat_interleave(2, 1), v.repeat_interleave(2, 1), is_causal=True)
    want = po(want.permute(0, 2, 1, 3).reshape(1, L, H * D).cuda().bfloat16())
    assert float((o.float() - want.float()).abs().max()) < 3e-2
    bad = torch.zeros(1, H, 1, D, device="cuda")
    with pytest.raises(TypeError):
        cm.append(bad, bad, bad, bad, bad, bad)
