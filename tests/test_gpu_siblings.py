"""The sink + window attention types and plain causal attention on the GPU, through the attention-type registry,
against oracle.siblings on the same bf16-rounded inputs (max-abs 2e-2 / mean-abs 2e-3)."""
import pytest
import torch

from oracle.rope import RopeOracle
from oracle.siblings import CausalOracle, SinkWindowOracle

pytestmark = pytest.mark.gpu

D, MAX_ABS, MEAN_ABS = 128, 2e-2, 2e-3


def _stream(T, H, Hkv, seed, B=1):
    g = torch.Generator().manual_seed(seed)
    mk = lambda h: torch.randn(B, T, h * D, generator=g).bfloat16()
    return mk(H), mk(Hkv), mk(Hkv)


def _drive(forward, x_q, x_k, x_v, calls, H, Hkv, base):
    """Call the attention type the way a patched decoder layer does, with identity projections."""
    from infllm_amd.attention import RotaryEmbeddingESM
    rope = RotaryEmbeddingESM(D, base=base, device="cuda")
    xq, xk, xv = x_q.cuda(), x_k.cuda(), x_v.cuda()
    past, outs, pos = None, [], 0
    for L in calls:
        sl = slice(pos, pos + L)
        kv = torch.cat((xk[:, sl], xv[:, sl]), dim=-1)
        o, past = forward(None, xq[:, sl], kv, rope, True, past, lambda t: t, lambda t: t[..., :Hkv * D], lambda t: t[..., Hkv * D:],
                          lambda t: t, D, H, Hkv)
        outs.append(o)
        pos += L
    torch.cuda.synchronize()
    return torch.cat(outs, dim=1).cpu(), past


def _heads(x, h):
    B, T, _ = x.shape
    return x.view(B, T, h, D).permute(0, 2, 1, 3).float()


def _check(got, want):
    B, H, T, _ = want.shape
    err = (got.float().view(B, T, H, D).permute(0, 2, 1, 3) - want).abs()
    assert float(err.max()) <= MAX_ABS and float(err.mean()) <= MEAN_ABS, (float(err.max()), float(err.mean()))


@pytest.mark.parametrize("kind", ["stream-llm", "infinite-lm"])
@pytest.mark.parametrize("calls,n_local,n_init", [([700], 256, 16), ([300, 1, 1, 1, 250, 47], 128, 8), ([1] * 40 + [90], 64, 4),
                                                  ([5, 200], 96, 0), ([150], 256, 16)])
def test_sink_window_types_follow_oracle(kind, calls, n_local, n_init):
    from infllm_amd.attention import ATTN_FORWRAD
    H, Hkv, T = 4, 2, sum(calls)
    xq, xk, xv = _stream(T, H, Hkv, seed=T + n_init, B=2)
    got, past = _drive(ATTN_FORWRAD[kind](n_local, n_init, fattn=False), xq, xk, xv, calls, H, Hkv, 1e4)
    ora = SinkWindowOracle(RopeOracle(D, base=1e4), n_local, n_init, kind)
    want, pos = [], 0
    for L in calls:
        sl = slice(pos, pos + L)
        want.append(ora.append(_heads(xq[:, sl], H), _heads(xk[:, sl], Hkv), _heads(xv[:, sl], Hkv)))
        pos += L
    _check(got, torch.cat(want, dim=2))
    assert past[2] == T and past[0].shape[2] == min(T, n_local + n_init) == past[1].shape[2]     # stream_llm.py:43-52


@pytest.mark.parametrize("kind", ["stream-llm", "infinite-lm", "origin"])
def test_sibling_types_with_heads_of_64(kind, monkeypatch):
    """head_dim 64 through the same three types: rows are widened for the kernels and cut back (attention/_rows.py)."""
    import sys
    from infllm_amd.attention import ATTN_FORWRAD
    monkeypatch.setattr(sys.modules[__name__], "D", 64)
    H, Hkv, calls, n_local, n_init = 4, 2, [300, 1, 1, 250], 128, 8
    T = sum(calls)
    xq, xk, xv = _stream(T, H, Hkv, seed=17, B=2)
    fwd = ATTN_FORWRAD[kind](False) if kind == "origin" else ATTN_FORWRAD[kind](n_local, n_init, fattn=False)
    got, past = _drive(fwd, xq, xk, xv, calls, H, Hkv, 1e4)
    ora = CausalOracle(RopeOracle(64, base=1e4)) if kind == "origin" else SinkWindowOracle(RopeOracle(64, base=1e4), n_local, n_init, kind)
    want, pos = [], 0
    for L in calls:
        sl = slice(pos, pos + L)
        want.append(ora.append(_heads(xq[:, sl], H), _heads(xk[:, sl], Hkv), _heads(xv[:, sl], Hkv)))
        pos += L
    _check(got, torch.cat(want, dim=2))
    assert past[0].shape[-1] == 64


def test_origin_type_is_causal_attention():
    from infllm_amd.attention import ATTN_FORWRAD
    H, Hkv, calls = 4, 4, [200, 1, 1, 130]
    T = sum(calls)
    xq, xk, xv = _stream(T, H, Hkv, seed=3)
    got, past = _drive(ATTN_FORWRAD["origin"](False), xq, xk, xv, calls, H, Hkv, 5e5)
    ora = CausalOracle(RopeOracle(D, base=5e5))
    want, pos = [], 0
    for L in calls:
        sl = slice(pos, pos + L)
        want.append(ora.append(_heads(xq[:, sl], H), _heads(xk[:, sl], Hkv), _heads(xv[:, sl], Hkv)))
        pos += L
    _check(got, torch.cat(want, dim=2))
    assert past[0].shape[2] == T


@pytest.mark.parametrize("pos0,consecutive", [(0, True), (777, True), (4095, False), (1000003, True)])
def test_rope_rows_matches_fp64_rotation(pos0, consecutive):
    from infllm_amd import ops
    B, H, L = 2, 3, 37
    g = torch.Generator().manual_seed(pos0 % 97)
    full = torch.randn(B, L + 5, H * D, generator=g).bfloat16()
    x = full.cuda()[:, 2:2 + L].view(B, L, H, D).permute(0, 2, 1, 3)          # strided rows, as the forwards pass them
    rope = RopeOracle(D, base=1e6)
    got = ops.rope_rows(x, rope.inv_freq.float().cuda(), 1.0, pos0, consecutive).cpu().double()
    xf = full[:, 2:2 + L].view(B, L, H, D).permute(0, 2, 1, 3).double()
    pos = torch.arange(L, dtype=torch.float64) * (1 if consecutive else 0) + pos0
    ang = pos[:, None] * rope.inv_freq.double()[None, :]
    lo, hi = xf[..., :D // 2], xf[..., D // 2:]
    want = torch.cat((lo * ang.cos() - hi * ang.sin(), hi * ang.cos() + lo * ang.sin()), dim=-1)
    assert float((got - want).abs().max()) <= 2 ** -7 * float(want.abs().max())      # one bf16 rounding
    empty = ops.rope_rows(x[:, :, :0], rope.inv_freq.float().cuda(), 1.0, 0)
    assert empty.shape == (B, H, 0, D)
