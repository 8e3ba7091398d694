"""The five benchmark configurations at their full sizes on the GPU.

A whole 131,072-token (let alone 1,048,576-token) stream is too long for the CPU oracle, so the long streams are
checked through (i) the closed forms of the state machine, (ii) byte-exact host copies of carved units, and (iii) the
oracle RESUMING from the state the GPU exported 20 execution blocks before the end (StreamOracle.from_state): both
sides then process the same last 10,240 tokens, and outputs, ordered selections, representative picks and the new
units' representatives are compared under the rules of tests/stream_parity.py.  Twenty blocks are more than two local
windows: the units carved in the last ten blocks consist of tokens that entered the stream after the snapshot, so
their whole score track (every block's joint softmax, 4096+ queries per token) is the oracle's own on the CPU side.
"""
import pytest
import torch

from stream_parity import (D, REFERENCE, REPR_TIE_REL, UNFAVOURED_GAP, Follower, assert_outputs_close, assert_reps_match, assert_tie_stats, compare, feed, make_stream,
                           new_manager, new_oracle)

pytestmark = pytest.mark.gpu

H, HKV = 32, 8
EXC, N_LOCAL, N_INIT, BS, TOPK = (REFERENCE[k] for k in ("exc_block_size", "n_local", "n_init", "block_size", "topk"))
RESUME_BLOCKS = 20


def _resume_in_oracle(cm, state, q_tail, k_tail, v_tail, calls, base, out_gpu, max_gap=UNFAVOURED_GAP):
    """The oracle continues from `state` over the tail tokens (CPU bf16 tensors) in the same calls the GPU made after the
    snapshot; cm must have recorded its trace over exactly those calls."""
    fol = Follower(cm, TOPK, REFERENCE["repr_topk"])
    ora = new_oracle(base, fol, **REFERENCE).from_state(state)
    first_new = ora.n_units
    outs, pos = [], 0
    for L in calls:
        sl = slice(pos, pos + L)
        outs.append(ora.append(q_tail[:, :, sl].float(), k_tail[:, :, sl].float(), v_tail[:, :, sl].float()))
        pos += L
    assert not fol.violations, fol.violations[:5]
    assert [b["order"] for b in cm.trace_blocks] == [b["order"] for b in ora.block_trace]
    assert len(ora.block_trace) == sum(-(-L // EXC) for L in calls)
    assert cm.num_global_block == ora.n_units and cm.length == ora.length
    assert_outputs_close(out_gpu, torch.cat(outs, dim=2))
    assert ora.n_units - first_new >= (sum(calls) - BS) // BS
    assert_reps_match(cm, ora, first_new)
    assert_tie_stats(fol, f"resumed over the last {sum(calls)} of {cm.length} tokens", max_gap)
    return ora, fol


@pytest.fixture(scope="module")
def stream_128k():
    q, k, v = make_stream(131072, H, HKV, seed=100)
    return q, k, v, q.cuda(), k.cuda(), v.cuda()


def test_config2_last_twenty_blocks_resume_in_the_oracle(stream_128k):
    """benchmark configuration 2 (131,072 tokens, bf16, mixture keys): closed forms of the state at the snapshot and at the
    end, then the last 20 execution blocks on both sides from the exported state."""
    q, k, v, qd, kd, vd = stream_128k
    T, base = 131072, 1e6
    T0 = T - RESUME_BLOCKS * EXC
    cm = new_manager(base, async_global_stream=True, **REFERENCE)
    pre = [8192] * (T0 // 8192) + ([T0 % 8192] if T0 % 8192 else [])
    feed(cm, qd, kd, vd, pre)
    state = cm.export_state()
    n_units = (T0 - N_INIT - N_LOCAL) // BS
    assert state["n_units"] == n_units == cm.num_global_block and state["init_len"] == N_INIT
    n_tail = state["tail_k"].shape[2]
    assert n_tail == T0 - N_INIT - n_units * BS and N_LOCAL <= n_tail < N_LOCAL + BS
    assert torch.equal(state["tail_k"].cpu(), k[:, :, T0 - n_tail:T0])
    assert torch.equal(state["init_v"].cpu(), v[:, :, :N_INIT])
    cm.record_trace = True
    calls = [T - T0 - 8192, 8192] if T - T0 > 8192 else [T - T0]
    got = torch.cat(feed(cm, qd, kd, vd, calls, pos=T0), dim=2).cpu()
    torch.cuda.synchronize()
    assert cm.length == T and cm.num_global_block == (T - N_INIT - N_LOCAL) // BS == 991
    ora, fol = _resume_in_oracle(cm, state, q[:, :, T0:], k[:, :, T0:], v[:, :, T0:], calls, base, got)
    assert fol.stats["selections"] == RESUME_BLOCKS and fol.stats["picks"] == H * (991 - n_units)
    for u in range(n_units, 991, 7):                            # carved units reached their pinned home
        lo = N_INIT + u * BS
        assert torch.equal(cm.host_unit(u)[0, 0], k[0, :, lo:lo + BS]) and torch.equal(cm.host_unit(u)[0, 1], v[0, :, lo:lo + BS]), u


def test_config2_stream_is_the_same_with_and_without_the_fetch_ahead(stream_128k, monkeypatch):
    """Config 2 at full size with 32 slots for 16 selected units of 512 KiB each: the stream with the fetch ahead of the
    selection (DMA engines, most guesses confirmed, the others repaired) against the stream without it - outputs bit for
    bit, hit / miss / eviction counts, the eviction sequence, the final residency, and the units' pinned host copies
    against the input.  Then against the stream whose selections run over all units instead of being ranked from the
    lists of their call: the same again, guesses included."""
    from infllm_amd.attention import ContextManager
    q, k, v, qd, kd, vd = stream_128k
    T = 131072
    monkeypatch.delenv("INFLLM_NO_DMA_FETCH", raising=False)      # the engines where the process can use them ...
    monkeypatch.delenv("INFLLM_NO_STAGING_COPY", raising=False)
    monkeypatch.setenv("INFLLM_FETCH_AHEAD_ALWAYS", "1")          # ... and guesses also where it cannot

    def run(ahead, lists=True):
        monkeypatch.setattr(ContextManager, "fetch_ahead", ahead)
        if lists:
            monkeypatch.delenv("INFLLM_NO_CALL_LISTS", raising=False)
        else:
            monkeypatch.setenv("INFLLM_NO_CALL_LISTS", "1")
        cm = new_manager(1e6, async_global_stream=True, **REFERENCE)
        outs = []
        for i, st in enumerate(range(0, T, 8192)):
            if i == 1:
                cm.policy[0].evicted_log = []
            outs.append(feed(cm, qd, kd, vd, [8192], pos=st)[0].cpu())
        torch.cuda.synchronize()
        return torch.cat(outs, dim=2), cm

    plain, cm0 = run(False)
    ahead, cm1 = run(True)
    issued, confirmed = cm1.prefetch_stats()
    assert cm0.prefetch_stats() == (0, 0) and issued > 200 and issued // 2 < confirmed < issued
    assert cm1.staged_units() > 20       # wrong guesses are the blocks in which a just-carved unit is selected: those came from staging
    assert torch.equal(plain, ahead)
    assert cm0.stats == cm1.stats and cm0.stats["misses"] > 3000
    assert cm0.policy[0].evicted_log == cm1.policy[0].evicted_log and cm0.policy[0].cached == cm1.policy[0].cached
    assert cm1.num_global_block == (T - N_INIT - N_LOCAL) // BS
    for u in range(0, cm1.num_global_block, 41):
        lo, hu = N_INIT + u * BS, cm1.host_unit(u)
        assert torch.equal(hu[0, 0], k[0, :, lo:lo + BS]) and torch.equal(hu[0, 1], v[0, :, lo:lo + BS]), u
    # ... and the same stream with every block's selection over all units instead of ranked from its call's lists
    every, cm2 = run(True, lists=False)
    assert cm1.path_counts()["call_ranked"] > 200 and cm2.path_counts()["call_ranked"] == 0
    assert torch.equal(every, ahead) and cm2.stats == cm1.stats and cm2.prefetch_stats() == cm1.prefetch_stats()
    assert cm2.policy[0].evicted_log == cm1.policy[0].evicted_log and cm2.policy[0].cached == cm1.policy[0].cached


def test_config1_literal_stream_follows_the_oracle():
    """benchmark configuration 1's workload on the HIP path: 16,384 tokens, q / k / v i.i.d. N(0,1) (rounded to bf16 once, the
    oracle consumes the same values in fp32), the whole stream on both sides.  With unstructured keys the unit scores
    crowd together, which is where the selection tie rule is exercised hardest."""
    T = 16384
    cm, ora, fol = compare(T, [8192, 8192], H=H, Hkv=HKV, base=1e6, seed=1, mixture=False, **REFERENCE)
    assert cm.num_global_block == (T - N_INIT - N_LOCAL) // BS == 95
    assert fol.stats["selections"] >= 15 and fol.stats["picks"] == 95 * H
    assert_tie_stats(fol, "config 1")


def test_config3_decode_steps_over_8192_units_follow_the_oracle():
    """benchmark configuration 3: a prepared memory of 8,192 units (1,048,576 past tokens) with representatives, then
    single-token steps.  Six steps are recomputed by the oracle from the same state: top-16 by brute force over all
    8,192 representatives, the fetch of the chosen units from pinned host memory, and the attention of one query."""
    import bench
    dev = torch.device("cuda:0")
    n_units, steps = 8192, 6
    state, tokens = bench.make_decode_state(dev, n_units, seed=3)
    cm = new_manager(1e6, async_global_stream=True, **REFERENCE).load_state(state)
    assert cm.num_global_block == n_units and cm.length == N_INIT + n_units * BS + N_LOCAL == state["length"]
    q, k, v = tokens(steps)
    cm.record_trace = True
    got = torch.cat(feed(cm, q, k, v, [1] * steps), dim=2).cpu()
    torch.cuda.synchronize()
    assert cm.stats["blocks"] == steps and cm.stats["misses"] > 0
    for u in (0, 4097, 8191):                                   # the prepared units sit in their pinned home
        assert torch.equal(cm.host_unit(u), state["units"][u].cpu())
    fol = Follower(cm, TOPK, REFERENCE["repr_topk"])
    ora = new_oracle(1e6, fol, **REFERENCE).from_state(state)
    qc, kc, vc = q.cpu().float(), k.cpu().float(), v.cpu().float()
    want = torch.cat([ora.append(qc[:, :, i:i + 1], kc[:, :, i:i + 1], vc[:, :, i:i + 1]) for i in range(steps)], dim=2)
    assert not fol.violations, fol.violations[:5]
    assert [b["order"] for b in cm.trace_blocks] == [b["order"] for b in ora.block_trace]
    assert all(len(b["order"][0]) == TOPK and b["n_units"] == n_units for b in ora.block_trace)
    assert_outputs_close(got, want)
    hits = sum(len(e["selected"]) - len(e["misses"]) for e in ora.cache[0].events)
    assert cm.stats["hits"] == hits and cm.stats["misses"] == steps * TOPK - hits
    assert_tie_stats(fol, "config 3")


def test_config5_million_token_stream_with_favoured_queries():
    """benchmark configuration 5: a 1,048,576-token stream whose queries lean towards 2 mixture components per execution
    block, max_cached_block 32, lru; evicted units live in pinned host memory and come back through the DMA engines.
    Closed forms (8,159 units), sampled host units byte for byte, hits and misses both present, and the last 20
    blocks - at positions around 10^6 - on both sides from the exported state."""
    import bench
    dev = torch.device("cuda:0")
    T, base = 1 << 20, 1e6
    qd, kd, vd = bench.make_stream(T, 5, dev, favour=2)
    T0 = T - RESUME_BLOCKS * EXC
    cm = new_manager(base, async_global_stream=True, **REFERENCE)
    pre = [8192] * (T0 // 8192) + ([T0 % 8192] if T0 % 8192 else [])
    feed(cm, qd, kd, vd, pre)
    state = cm.export_state(with_units=False)
    n_units = (T0 - N_INIT - N_LOCAL) // BS
    assert state["n_units"] == n_units == cm.num_global_block
    assert cm.stats["misses"] > 1000 and cm.stats["hits"] > 1000 and cm.stats["evictions"] > 1000
    # a block selects min(topk, units carved before it) units; every one of them is a hit or a miss
    assert cm.stats["hits"] + cm.stats["misses"] == sum(min(TOPK, max(0, (b * EXC - N_INIT - N_LOCAL) // BS)) for b in range(T0 // EXC))

    class HostUnits:                                            # the units where they live: pinned host memory
        def __getitem__(self, u):
            return cm.host_unit(u)

    state["units"] = HostUnits()
    cm.record_trace = True
    calls = [T - T0 - 8192, 8192]
    got = torch.cat(feed(cm, qd, kd, vd, calls, pos=T0), dim=2).cpu()
    torch.cuda.synchronize()
    assert cm.length == T and cm.num_global_block == (T - N_INIT - N_LOCAL) // BS == 8159
    for u in list(range(0, 8159, 509)) + [8158]:
        lo, hu = N_INIT + u * BS, cm.host_unit(u)
        assert torch.equal(hu[0, 0], kd[0, :, lo:lo + BS].cpu()) and torch.equal(hu[0, 1], vd[0, :, lo:lo + BS].cpu()), u
    tail = slice(T0, T)
    # favoured queries put a token's mass on a few near-one probabilities: the picks get the full rule (stream_parity.py)
    _resume_in_oracle(cm, state, qd[:, :, tail].cpu(), kd[:, :, tail].cpu(), vd[:, :, tail].cpu(), calls, base, got, max_gap=REPR_TIE_REL)
