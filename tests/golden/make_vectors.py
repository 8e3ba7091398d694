"""Writes tests/golden/oracle_small.npz: outputs of the CPU oracle on small seeded inputs.

The reference ships no tests, fixtures or golden vectors for this path and was never executed, so these are NOT
reference outputs: they freeze what oracle/ computed when its mathematical pins (tests/test_oracle_*.py) passed,
so that a later edit of the oracle that changes results is noticed even if it happens to keep the pins green.
Inputs are regenerated from the seeds below; only the expected outputs are stored.

Run from the repository root:  python tests/golden/make_vectors.py
"""
import os
import sys

import numpy as np
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)

from oracle.rope import RopeOracle                      # noqa: E402
from oracle.siblings import SinkWindowOracle            # noqa: E402
from oracle.stream import StreamOracle                  # noqa: E402

GEOM = dict(n_init=4, n_local=32, block_size=8, max_cached_block=4, topk=2, exc_block_size=16, repr_topk=2)
CALLS = [70, 1, 1, 48, 31]


def inputs(seed, T, H=4, Hkv=2, D=16):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(1, H, T, D, generator=g), torch.randn(1, Hkv, T, D, generator=g),
            torch.randn(1, Hkv, T, D, generator=g))


def run(oracle, q, k, v, calls):
    outs, pos = [], 0
    for L in calls:
        outs.append(oracle.append(q[:, :, pos:pos + L], k[:, :, pos:pos + L], v[:, :, pos:pos + L]))
        pos += L
    return torch.cat(outs, dim=2)


def vectors():
    T = sum(CALLS)
    q, k, v = inputs(1234, T)
    out = {}
    for name, extra in (("lru", {}), ("lru_s", dict(cache_strategy="lru-s", score_decay=0.1)),
                        ("chunk", dict(chunk_topk_calc=32))):
        cm = StreamOracle(RopeOracle(16, base=10000), **GEOM, **extra)
        out[f"stream_{name}_out"] = run(cm, q, k, v, CALLS).numpy()
        out[f"stream_{name}_selected"] = np.array([b["selected"][0] + [-1] * (GEOM["topk"] - len(b["selected"][0]))
                                                    for b in cm.block_trace], dtype=np.int32)
        out[f"stream_{name}_evicted"] = np.array([len(e["evicted"]) for e in cm.cache[0].events], dtype=np.int32)
    for kind in ("stream-llm", "infinite-lm"):
        out[f"sink_{kind}_out"] = run(SinkWindowOracle(RopeOracle(16, base=10000), 24, 4, kind), q, k, v, CALLS).numpy()
    return out


if __name__ == "__main__":
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "oracle_small.npz")
    np.savez_compressed(path, **vectors())
    print("wrote", path, os.path.getsize(path), "bytes")
