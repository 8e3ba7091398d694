"""Pins for oracle.siblings (restating stream_llm.py, infinite_lm.py, origin.py).

The reference holds no tests or fixtures for these attention types; the per-call restatement is pinned against
a dense derivation in absolute positions, an explicit fp64 complex-rotation loop on a tiny case, and the
reductions to causal / banded scaled-dot-product attention.
"""
import cmath
import math

import pytest
import torch
import torch.nn.functional as F

from oracle.rope import RopeOracle
from oracle.siblings import CausalOracle, SinkWindowOracle, sink_window_dense


def _stream(T, H=4, Hkv=2, D=16, seed=0, B=1):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(B, H, T, D, generator=g), torch.randn(B, Hkv, T, D, generator=g),
            torch.randn(B, Hkv, T, D, generator=g))


def _run(ora, q, k, v, calls):
    outs, pos = [], 0
    for L in calls:
        outs.append(ora.append(q[:, :, pos:pos + L], k[:, :, pos:pos + L], v[:, :, pos:pos + L]))
        pos += L
    return torch.cat(outs, dim=2)


@pytest.mark.parametrize("kind", ["stream-llm", "infinite-lm"])
@pytest.mark.parametrize("calls", [[90], [40, 1, 1, 30, 18], [1] * 50, [3, 60, 27]])
def test_per_call_restatement_equals_dense_absolute_derivation(kind, calls):
    T = sum(calls)
    q, k, v = _stream(T, seed=len(calls))
    rope = RopeOracle(16, base=10000)
    got = _run(SinkWindowOracle(rope, 24, 4, kind), q, k, v, calls)
    want = sink_window_dense(q[0], k[0], v[0], rope, 24, 4, kind)
    assert torch.allclose(got[0].double(), want, atol=2e-4), float((got[0].double() - want).abs().max())


@pytest.mark.parametrize("kind", ["stream-llm", "infinite-lm"])
def test_dense_derivation_against_explicit_complex_rotation(kind):
    """Tiny case, every logit from first principles: pair (d, d + D/2) is the complex number x_d + i x_{d+D/2},
    rotating by angle a multiplies it by e^{ia}; q.k = Re sum conj-free product of the rotated vectors."""
    T, D, n_local, n_init, base = 9, 8, 4, 2, 100.0
    q, k, v = _stream(T, H=1, Hkv=1, D=D, seed=5)
    q, k, v = q[0, 0].double(), k[0, 0].double(), v[0, 0].double()
    freq = [base ** (-2 * i / D) for i in range(D // 2)]

    def rot(x, position):
        z = [complex(x[d], x[d + D // 2]) * cmath.exp(1j * position * freq[d]) for d in range(D // 2)]
        return [c.real for c in z] + [c.imag for c in z]

    out = torch.zeros(T, D, dtype=torch.float64)
    for p in range(T):
        logit, keys = [], []
        for j in range(p + 1):
            if p - j < n_local:
                a, b = rot(q[p], p), rot(k[j], j)
            elif j < n_init:
                if kind == "infinite-lm":
                    a, b = rot(q[p], n_local - 1), list(k[j])
                else:
                    a, b = rot(q[p], n_local + n_init - 1), rot(k[j], j)
            else:
                continue
            logit.append(sum(float(x) * float(y) for x, y in zip(a, b)) / math.sqrt(D))
            keys.append(j)
        m = max(logit)
        w = [math.exp(x - m) for x in logit]
        for wj, j in zip(w, keys):
            out[p] += wj / sum(w) * v[j]
    rope = RopeOracle(D, base=base)
    dense = sink_window_dense(q[None].float(), k[None].float(), v[None].float(), rope, n_local, n_init, kind)[0]
    assert torch.allclose(dense, out, atol=1e-5)
    stateful = _run(SinkWindowOracle(rope, n_local, n_init, kind), q[None, None].float(), k[None, None].float(),
                    v[None, None].float(), [4, 1, 4])[0, 0]
    assert torch.allclose(stateful.double(), out, atol=1e-4)


def _sdpa(q, k, v, mask):
    G = q.shape[1] // k.shape[1]
    return F.scaled_dot_product_attention(q, k.repeat_interleave(G, dim=1), v.repeat_interleave(G, dim=1), attn_mask=mask)


@pytest.mark.parametrize("kind", ["stream-llm", "infinite-lm"])
def test_reductions_to_library_attention(kind):
    T = 60
    q, k, v = _stream(T, seed=9)
    rope = RopeOracle(16)
    pos = list(range(T))
    qa, ka = rope.rotate(q, pos), rope.rotate(k, pos)
    dist = torch.arange(T)[:, None] - torch.arange(T)[None, :]
    # stream inside the window: causal attention with standard RoPE
    got = _run(SinkWindowOracle(rope, 64, 4, kind), q, k, v, [20, 40])
    assert torch.allclose(got, _sdpa(qa, ka, v, dist >= 0), atol=2e-5)
    # no sinks: banded attention
    got = _run(SinkWindowOracle(rope, 16, 0, kind), q, k, v, [20, 1, 39])
    assert torch.allclose(got, _sdpa(qa, ka, v, (dist >= 0) & (dist < 16)), atol=2e-5)


def test_causal_oracle_is_sdpa_with_rope_and_ignores_call_splitting():
    T = 50
    q, k, v = _stream(T, seed=11, B=2)
    rope = RopeOracle(16)
    pos = list(range(T))
    want = _sdpa(rope.rotate(q, pos), rope.rotate(k, pos), v, torch.arange(T)[:, None] >= torch.arange(T)[None, :])
    for calls in ([50], [17, 1, 1, 31], [1] * 50):
        assert torch.allclose(_run(CausalOracle(rope), q, k, v, calls), want, atol=2e-5)
