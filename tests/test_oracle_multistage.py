"""Pins for oracle.multistage (restating torch_impl.py): library softmax / SDPA and brute force."""
import math

import torch
import torch.nn.functional as F

from oracle.multistage import MultiStageOracle, stage_mask, expand_kv


def _loops(q, ks, vs, vis_fns):
    """Pure-Python joint softmax over stages; q [H,Lq,D], ks[s] [Hkv,Lk,D]."""
    H, Lq, D = q.shape
    out = torch.zeros(H, Lq, D, dtype=torch.float64)
    scores = [torch.zeros(H, k.shape[1], dtype=torch.float64) for k in ks]
    for h in range(H):
        for i in range(Lq):
            terms = []
            for s, (k, v, vis) in enumerate(zip(ks, vs, vis_fns)):
                g = h // (H // k.shape[0])
                for j in range(k.shape[1]):
                    if vis(i, j):
                        terms.append((s, j, float(q[h, i].double() @ k[g, j].double()) / math.sqrt(D), v[g, j].double()))
            m = max(t[2] for t in terms)
            den = sum(math.exp(t[2] - m) for t in terms)
            for s, j, lg, vv in terms:
                p = math.exp(lg - m) / den
                out[h, i] += p * vv
                scores[s][h, j] += p
    return out, scores


def test_two_stage_equals_brute_force_loops():
    torch.manual_seed(0)
    H, Hkv, Lq, D, L1, L2, w = 4, 2, 5, 8, 9, 6, 4
    q = torch.randn(1, H, Lq, D)
    k1, v1 = torch.randn(1, Hkv, L1, D), torch.randn(1, Hkv, L1, D)
    k2, v2 = torch.randn(1, Hkv, L2, D), torch.randn(1, Hkv, L2, D)
    a = MultiStageOracle(q.shape)
    a.append(q, k1, v1, sliding_window=w, get_score=True)
    a.append(q, k2, v2, sliding_window=(3, w), complement_sliding_window=True, end=True, get_score=True)
    out, (s1, s2) = a.get_result()
    off1 = L1 - Lq
    want, (w1, w2) = _loops(q[0], [k1[0], k2[0]], [v1[0], v2[0]],
                            [lambda i, j: 0 <= i - j + off1 < w, lambda i, j: i - j + 3 >= w])
    assert torch.allclose(out[0].double(), want, atol=1e-5)
    assert torch.allclose(s1[0].double(), w1, atol=1e-5)
    assert torch.allclose(s2[0].double(), w2, atol=1e-5)


def test_equals_sdpa_on_concatenated_keys():
    torch.manual_seed(1)
    H, Hkv, Lq, D, L1, L2, w = 6, 3, 16, 16, 40, 24, 20
    q = torch.randn(2, H, Lq, D)
    k1, v1 = torch.randn(2, Hkv, L1, D), torch.randn(2, Hkv, L1, D)
    k2, v2 = torch.randn(2, Hkv, L2, D), torch.randn(2, Hkv, L2, D)
    a = MultiStageOracle(q.shape)
    a.append(q, k1, v1, sliding_window=w, get_score=True)
    a.append(q, k2, v2, end=True)
    out, (s1, s2) = a.get_result()
    assert s2 is None
    mask = torch.cat((stage_mask(Lq, L1, w), torch.ones(Lq, L2, dtype=torch.bool)), dim=-1)
    kk = torch.cat((expand_kv(k1, H), expand_kv(k2, H)), dim=-2)
    vv = torch.cat((expand_kv(v1, H), expand_kv(v2, H)), dim=-2)
    want = F.scaled_dot_product_attention(q, kk, vv, attn_mask=mask)
    assert torch.allclose(out, want, atol=1e-5)
    p = torch.softmax((q @ kk.transpose(-1, -2) / math.sqrt(D)).masked_fill(~mask, float("-inf")), dim=-1)
    assert torch.allclose(s1, p[..., :L1].sum(dim=-2), atol=1e-5)
    # probabilities of one query over all stages sum to one
    assert torch.allclose(p.sum(-1), torch.ones(2, H, Lq), atol=1e-5)


def test_int_window_is_right_aligned_causal_band():
    m = stage_mask(3, 6, 2)
    want = torch.tensor([[0, 0, 1, 1, 0, 0], [0, 0, 0, 1, 1, 0], [0, 0, 0, 0, 1, 1]], dtype=torch.bool)
    assert torch.equal(m, want)
    assert torch.equal(stage_mask(3, 6, (3, 2)), want)
    comp = stage_mask(3, 6, (3, 2), complement=True)
    assert torch.equal(comp, torch.tensor([[1, 1, 0, 0, 0, 0], [1, 1, 1, 0, 0, 0], [1, 1, 1, 1, 0, 0]], dtype=torch.bool))


def test_single_causal_stage_is_causal_sdpa():
    torch.manual_seed(2)
    q, k, v = torch.randn(1, 2, 12, 8), torch.randn(1, 2, 12, 8), torch.randn(1, 2, 12, 8)
    a = MultiStageOracle(q.shape)
    a.append(q, k, v, sliding_window=64, end=True)
    assert torch.allclose(a.get_result()[0], F.scaled_dot_product_attention(q, k, v, is_causal=True), atol=1e-5)


def test_global_keys_are_permutation_invariant():
    torch.manual_seed(3)
    q = torch.randn(1, 2, 4, 8)
    k1, v1 = torch.randn(1, 2, 6, 8), torch.randn(1, 2, 6, 8)
    k2, v2 = torch.randn(1, 2, 10, 8), torch.randn(1, 2, 10, 8)
    perm = torch.randperm(10)
    outs = []
    for kk, vv in ((k2, v2), (k2[:, :, perm], v2[:, :, perm])):
        a = MultiStageOracle(q.shape)
        a.append(q, k1, v1, sliding_window=5, get_score=True)
        a.append(q, kk, vv, end=True)
        outs.append(a.get_result())
    assert torch.allclose(outs[0][0], outs[1][0], atol=1e-6)
    assert torch.allclose(outs[0][1][0], outs[1][1][0], atol=1e-6)


def test_empty_second_stage():
    torch.manual_seed(4)
    q, k, v = torch.randn(1, 2, 3, 8), torch.randn(1, 1, 3, 8), torch.randn(1, 1, 3, 8)
    a = MultiStageOracle(q.shape)
    a.append(q, k, v, sliding_window=8)
    a.append(q, k[:, :, :0], v[:, :, :0], end=True, sliding_window=(0, 8), complement_sliding_window=True)
    want = F.scaled_dot_product_attention(q, expand_kv(k, 2), expand_kv(v, 2), is_causal=True)
    assert torch.allclose(a.get_result()[0], want, atol=1e-5)
