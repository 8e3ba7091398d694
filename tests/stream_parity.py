"""Shared machinery of the GPU stream-parity tests: seeded streams, the GPU run, and the Follower that lets the CPU
oracle adopt the GPU's discrete choices where the acceptance rule allows them to differ.

Acceptance rules (written here once, used by every stream test):

* outputs: max-abs 2e-2 / mean-abs 2e-3 against the fp32 oracle on the same bf16-rounded inputs;
* retrieved unit sets: identical to the oracle's, except that a unit may be swapped for another whose oracle score
  lies within TIE_REL = 1e-3 relative of the k-th score; the ORDER of a selection (torch.topk order, which the
  residency policy sees) may differ from the oracle's only between neighbours whose oracle scores are within TIE_REL;
* representative keys (the repr_topk best tokens of a unit per query head): a pick may differ from the oracle's only
  if the oracle's scores of the swapped tokens lie within REPR_TIE_REL = 1e-2 relative of the repr_topk-th score.  The
  token scores are sums of bf16-MFMA probabilities (rotated q and k are rounded to bf16 once, 2^-9 relative each, as
  the reference's bf16 runs round them), so the score of a token whose mass comes from few queries moves by a few
  1e-3.  Measured: over 18,560 picks of unfavoured streams (20 of the small geometry, 10 of the reference geometry,
  N(0,1) and mixture keys) plus the 2,880 picks of the two-layer Llama-3-8B-shaped model 1.5 % of the picks differ at
  all, 15 of them by more than 1e-3, the largest gaps being 1.19e-3 (mixture keys), 1.40e-3 (N(0,1) keys), 2.05e-3
  (small geometry) and 2.09e-3 (model activations); such streams are held to UNFAVOURED_GAP = 4e-3, twice the
  largest.  benchmark configuration 5 is the wide one: its queries lean towards two mixture components per block, so a token's
  mass comes from a handful of near-one probabilities - 19 of 2,560 picks differ, 14 by more than 1e-3, five beyond
  4e-3, the largest 6.29e-3 (the same with the score kernel of either form, bit for bit); it is held to the full 1e-2.
  How often a pick differs at all, and by more than 1e-3, is counted (Follower.stats), bounded for every stream by
  assert_tie_stats() and in total by the sweep in test_gpu_stream.py.

Where a choice differs within its rule the oracle adopts the GPU's (topk_hook / repr_hook), so that the two
trajectories stay comparable: every later decision is then judged on the same history.  The oracle keeps its
representatives in bf16 (rep_dtype), as the reference's bf16 runs do (context_manager.py:321-328).
"""
import torch

from oracle.rope import RopeOracle
from oracle.stream import StreamOracle

MAX_ABS, MEAN_ABS = 2e-2, 2e-3
TIE_REL, REPR_TIE_REL = 1e-3, 1e-2
UNFAVOURED_GAP = 4e-3
D = 128

SMALL = dict(n_init=16, n_local=256, block_size=32, max_cached_block=8, topk=4, exc_block_size=64, repr_topk=2)
REFERENCE = dict(n_init=128, n_local=4096, block_size=128, max_cached_block=32, topk=16, exc_block_size=512, repr_topk=4)


def make_stream(T, H, Hkv, seed, B=1, mixture=True, D=D):
    """q, v ~ N(0,1); keys from a 64-component Gaussian mixture (std 0.3 around N(0,1) means), or N(0,1)."""
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


def new_manager(base, **kw):
    from infllm_amd.attention import ContextManager, RotaryEmbeddingESM
    rope = RotaryEmbeddingESM(kw.get("dim", D), base=base, device="cuda")
    return ContextManager(rope, kw["n_init"], kw["n_local"], kw["block_size"], kw["max_cached_block"], kw["topk"],
                          kw["exc_block_size"], kw.get("score_decay"), False, kw.get("repr_topk", 1),
                          kw.get("cache_strategy", "lru"), kw.get("chunk_topk_calc"), kw.get("async_global_stream", False), False, False,
                          kw.get("perhead", False))


def feed(cm, qd, kd, vd, calls, pos=0):
    """append() the device tensors in calls of the given lengths, starting at position `pos` of the tensors."""
    outs = []
    for L in calls:
        sl = slice(pos, pos + L)
        outs.append(cm.append(qd[:, :, sl], kd[:, :, sl], vd[:, :, sl], qd[:, :, sl], kd[:, :, sl], vd[:, :, sl]))
        pos += L
    return outs


def run_gpu(q, k, v, calls, base, **kw):
    cm = new_manager(base, **kw)
    cm.record_trace = True
    outs = feed(cm, q.cuda(), k.cuda(), v.cuda(), calls)
    torch.cuda.synchronize()
    return torch.cat(outs, dim=2).cpu(), cm


def new_oracle(base, follower=None, **kw):
    return StreamOracle(RopeOracle(kw.get("dim", D), base=base), kw["n_init"], kw["n_local"], kw["block_size"], kw["max_cached_block"],
                        kw["topk"], kw["exc_block_size"], repr_topk=kw.get("repr_topk", 1), perhead=kw.get("perhead", False),
                        topk_hook=follower.topk_hook if follower else None, repr_hook=follower.repr_hook if follower else None,
                        cache_strategy=kw.get("cache_strategy", "lru"), score_decay=kw.get("score_decay"),
                        chunk_topk_calc=kw.get("chunk_topk_calc"), rep_dtype=torch.bfloat16)


class Follower:
    """Oracle hooks that adopt the GPU's choices when the tie rules allow it, and count how often they had to."""

    def __init__(self, cm, topk, repr_topk):
        self.blocks = cm.trace_blocks
        self.repr = cm.trace_repr_indices()
        self.topk, self.repr_topk = topk, repr_topk
        self.violations = []
        self.stats = dict(selections=0, tie_topk=0, order_swaps=0, picks=0, tie_repr=0, repr_beyond_1e3=0, repr_max_gap=0.0)
        self.repr_gaps = []           # relative gap of every pick that differs from the oracle's

    def topk_hook(self, block, row, scores):
        st = self.stats
        st["selections"] += 1
        gpu_order = list(self.blocks[block]["order"][row])
        top = scores.topk(self.topk)
        mine_order = top.indices.tolist()
        if gpu_order == mine_order:
            return None
        gpu, mine = set(gpu_order), set(mine_order)
        kth = float(top.values[-1])
        if gpu != mine:
            bad = [i for i in gpu ^ mine if abs(float(scores[i]) - kth) > TIE_REL * abs(kth)]
            if bad:
                self.violations.append(("topk", block, row, bad))
            st["tie_topk"] += 1
        # the GPU's order against the oracle's scores: a score may rise from one entry to the next only within the tie rule
        vals = [float(scores[i]) for i in gpu_order]
        for a, b in zip(vals[:-1], vals[1:]):
            if b - a > TIE_REL * max(abs(a), abs(b)):
                self.violations.append(("order", block, row, gpu_order, vals))
                break
        if gpu == mine:
            st["order_swaps"] += 1
        return gpu_order

    def repr_hook(self, unit, row, score):
        st = self.stats
        gpu = self.repr[unit][row].long()                      # [H, r]
        mine = score.topk(self.repr_topk, dim=-1)
        for h in range(score.shape[0]):
            st["picks"] += 1
            a, b = set(gpu[h].tolist()), set(mine.indices[h].tolist())
            if a != b:
                rth = float(mine.values[h, -1])
                gaps = [abs(float(score[h, i]) - rth) / max(abs(rth), 1e-30) for i in a ^ b]
                if max(gaps) > REPR_TIE_REL:
                    self.violations.append(("repr", unit, row, h, sorted(a ^ b), max(gaps)))
                st["tie_repr"] += 1
                self.repr_gaps.append(max(gaps))
                st["repr_beyond_1e3"] += max(gaps) > TIE_REL
                st["repr_max_gap"] = max(st["repr_max_gap"], max(gaps))
        return gpu


def assert_tie_stats(fol, what, max_gap=UNFAVOURED_GAP):
    """Print how often the tie rules were used on one stream and bound it: picks that differ at all <= 4 %, by more
    than 1e-3 <= 1 %, none beyond max_gap (REPR_TIE_REL itself is a violation); selections that differ in set or order
    <= 10 % (at least two are allowed: streams of twenty selections)."""
    st = fol.stats
    print(f"{what}: {st}")
    assert not fol.violations, fol.violations[:5]
    assert st["repr_max_gap"] <= max_gap, (what, st)
    assert st["tie_repr"] <= max(2, 0.04 * st["picks"]) and st["repr_beyond_1e3"] <= max(2, 0.01 * st["picks"]), (what, st)
    assert st["tie_topk"] + st["order_swaps"] <= max(2, 0.10 * st["selections"]), (what, st)


def assert_outputs_close(got, want, what="", relative_above_one=False):
    """max-abs / mean-abs of the acceptance rule.  relative_above_one: the max-abs bound becomes MAX_ABS * |want| for
    outputs beyond 1 in magnitude - for inputs that are not N(0,1) (activations of a decoder reach |v| = 7 and attention
    rows that rest on one or two keys give outputs of 2..5, where neighbouring bf16 values are 0.016 or 0.031 apart, so
    the rounding of the bf16 result alone can use up an absolute 2e-2)."""
    err = (got.float() - want.float()).abs()
    worst = err / want.float().abs().clamp_min(1.0) if relative_above_one else err
    assert float(worst.max()) <= MAX_ABS and float(err.mean()) <= MEAN_ABS, (what, float(worst.max()), float(err.max()), float(err.mean()))


def assert_reps_match(cm, ora, first_unit=0):
    """The GPU's representatives of units [first_unit, n) against the oracle's (which follow the same picks): equal up
    to one bf16 rounding (the fp32 sums of repr_topk keys may be formed in a different order)."""
    n = ora.n_units
    if n <= first_unit:
        return
    for u in range(len(ora.reps)):
        want = torch.stack(ora.reps[u][first_unit:n]).float()
        got = cm.rep_rows(u, first_unit, n)
        tol = 2.0 ** -7 * torch.maximum(want.abs(), got.abs()) + 1e-30
        assert bool(((got - want).abs() <= tol).all()), (u, float((got - want).abs().max()))


def follow(cm, got, q, k, v, calls, base, relative_above_one=False, **kw):
    """The oracle over the CPU bf16 tensors q, k, v in the given calls, following the choices of `cm` (a manager that
    recorded its trace over exactly those calls and returned `got`); asserts every rule above and returns
    (oracle, follower)."""
    fol = Follower(cm, kw["topk"], kw.get("repr_topk", 1))
    ora = new_oracle(base, fol, **kw)
    outs, pos = [], 0
    for L in calls:
        sl = slice(pos, pos + L)
        outs.append(ora.append(q[:, :, sl].float(), k[:, :, sl].float(), v[:, :, sl].float()))
        pos += L
    want = torch.cat(outs, dim=2)
    assert not fol.violations, fol.violations[:5]
    assert [b["order"] for b in cm.trace_blocks] == [b["order"] for b in ora.block_trace]
    assert cm.num_global_block == ora.n_units and cm.length == ora.length == pos
    assert_outputs_close(got, want, relative_above_one=relative_above_one)
    if not kw.get("perhead", False):
        assert_reps_match(cm, ora)
        # the cache model saw the same ordered selections, so residency events must match too
        hits = sum(len(e["selected"]) - len(e["misses"]) for c in ora.cache for e in c.events)
        assert cm.stats["hits"] == hits
        assert cm.stats["evictions"] == sum(len(e["evicted"]) for c in ora.cache for e in c.events)
    return ora, fol


def compare(T, calls, H, Hkv, base, seed, B=1, mixture=True, **kw):
    """One stream through the GPU ContextManager and through the oracle following it; returns (cm, oracle, follower)."""
    q, k, v = make_stream(T, H, Hkv, seed, B=B, mixture=mixture, D=kw.get("dim", D))
    got, cm = run_gpu(q, k, v, calls, base, **kw)
    assert sum(calls) == T
    ora, fol = follow(cm, got, q, k, v, calls, base, **kw)
    return cm, ora, fol
