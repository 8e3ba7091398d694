"""GPU parity of every kernel entry point (called through the C ABI) against the CPU oracle.

Acceptance (floating point): attention outputs within max-abs 2e-2 / mean-abs 2e-3 of
the fp32 oracle evaluated on the same bf16-rounded inputs; index outputs exact except
where two candidates' oracle scores are within 1e-3 relative of each other.
"""
import math

import numpy as np
import pytest
import torch

from oracle.multistage import MultiStageOracle
from oracle.rope import RopeOracle

pytestmark = pytest.mark.gpu

MAX_ABS, MEAN_ABS = 2e-2, 2e-3
D = 128


def _ops():
    from infllm_amd import ops
    return ops


def _rand(shape, seed, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(shape, generator=g) * scale).bfloat16()


def _check_out(got, want, what=""):
    err = (got.float().cpu() - want.float()).abs()
    assert float(err.max()) <= MAX_ABS and float(err.mean()) <= MEAN_ABS, (what, float(err.max()), float(err.mean()))


# ------------------------------------------------------------------ prologue
@pytest.mark.parametrize("pos0,n", [(0, 40), (4090, 17), (1_000_003, 33), (2 ** 31 + 5, 8)])
def test_ingest_matches_rope_oracle(pos0, n):
    ops = _ops()
    B, H, Hkv, cap, n_local = 2, 4, 2, 128, 4096
    q, k, v = _rand((B, H, n, D), 1), _rand((B, Hkv, n, D), 2), _rand((B, Hkv, n, D), 3)
    rope = RopeOracle(D, base=1e6)
    dev = "cuda"
    rk_raw = torch.zeros((B, Hkv, cap, D), dtype=torch.bfloat16, device=dev)
    rk_rot, rv = torch.zeros_like(rk_raw), torch.zeros_like(rk_raw)
    rscore = torch.ones((B, H, cap), dtype=torch.float32, device=dev)
    q_loc = torch.zeros((B, H, n, D), dtype=torch.bfloat16, device=dev)
    q_glb = torch.zeros_like(q_loc)
    # strided inputs ([B, n, heads, D] memory order) exercise the stride arguments
    qd = q.permute(0, 2, 1, 3).contiguous().to(dev).permute(0, 2, 1, 3)
    ops.ingest(qd, k.to(dev), v.to(dev), pos0, n_local - 1, rope.inv_freq.to(dev), 1.0, rk_raw, rk_rot, rv, rscore, q_loc, q_glb)
    torch.cuda.synchronize()
    rows = [(pos0 + i) % cap for i in range(n)]
    assert torch.equal(rk_raw[:, :, rows].cpu(), k) and torch.equal(rv[:, :, rows].cpu(), v)
    assert float(rscore[:, :, rows].abs().max()) == 0.0
    untouched = [r for r in range(cap) if r not in rows]
    assert float(rscore[:, :, untouched].min()) == 1.0 and float(rk_raw[:, :, untouched].abs().max()) == 0.0
    # fp64 rotation with the reference's fp32 inverse frequencies
    inv = rope.inv_freq.double()
    ang = torch.arange(pos0, pos0 + n, dtype=torch.float64)[:, None] * inv[None, :]

    def rot(x, ang):
        xd = x.double()
        lo, hi = xd[..., :64], xd[..., 64:]
        return torch.cat((lo * ang.cos() - hi * ang.sin(), hi * ang.cos() + lo * ang.sin()), dim=-1)

    for got, src, a in ((q_loc, q, ang), (rk_rot[:, :, rows], k, ang),
                        (q_glb, q, torch.full((n, 1), float(n_local - 1), dtype=torch.float64) * inv[None, :])):
        want = rot(src, a)
        ulp = want.abs().clamp_min(2.0 ** -126) * 2.0 ** -8          # half a bf16 ulp, relative, plus slack
        assert bool(((got.cpu().double() - want).abs() <= ulp * 1.01 + 1e-6).all())
    if pos0 + n < 10000:     # small positions (fp32 angles still exact enough): equal to the fp32 oracle up to one bf16 rounding
        want = rope.rotate(q.float(), list(range(pos0, pos0 + n)))
        assert float((q_loc.cpu().float() - want).abs().max()) <= 2.0 ** -7 * float(want.abs().max())


def test_ingest_partial_sums_give_the_mean_global_query():
    ops = _ops()
    B, H, Hkv, n, cap = 2, 8, 2, 77, 128
    q, k, v = _rand((B, H, n, D), 5), _rand((B, Hkv, n, D), 6), _rand((B, Hkv, n, D), 7)
    rope = RopeOracle(D, base=1e4)
    z = lambda *s: torch.zeros(s, dtype=torch.bfloat16, device="cuda")
    rk_raw, rk_rot, rv = z(B, Hkv, cap, D), z(B, Hkv, cap, D), z(B, Hkv, cap, D)
    rscore = torch.zeros((B, H, cap), dtype=torch.float32, device="cuda")
    q_loc, q_glb = z(B, H, n, D), z(B, H, n, D)
    qpart = torch.full((B, (n + 15) // 16, H * D), 9.0, dtype=torch.float32, device="cuda")
    ops.ingest(q.cuda(), k.cuda(), v.cuda(), 3, 63, rope.inv_freq.cuda(), 1.0, rk_raw, rk_rot, rv, rscore, q_loc, q_glb, qpart)
    qbar = torch.zeros((B, H * D), dtype=torch.float32, device="cuda")
    ops.reduce_partials(qpart, 1.0 / n, qbar)
    # the sums are taken before q_glb is rounded to bf16: the mean query is the fp32 oracle's up to fp32 rounding,
    # and the bf16 rows' own mean differs from it by their rounding (2^-9 relative per element, averaged down)
    want = rope.one_angle(q.float(), 64).mean(dim=2).reshape(B, H * D)
    assert torch.allclose(qbar.cpu(), want, atol=2e-6)
    assert torch.allclose(q_glb.float().mean(dim=2).reshape(B, H * D).cpu(), want, atol=2e-3)


def test_block_mean():
    ops = _ops()
    B, H, n, exc = 2, 3, 70, 32
    x = _rand((B, H, n, D), 4).cuda()
    qbar = torch.zeros((B, 3, H * D), dtype=torch.float32, device="cuda")
    ops.block_mean(x, B, H, n, exc, qbar)
    xf = x.float()
    for j, (a, b) in enumerate(((0, 32), (32, 64), (64, 70))):
        want = xf[:, :, a:b].mean(dim=2).reshape(B, H * D)
        assert torch.allclose(qbar[:, j], want, atol=1e-5)


def test_chunk_qbar_is_the_mean_of_the_one_angle_rotation():
    """infllm_chunk_qbar means first and rotates once; the oracle rotates every row (rope.py:93-104) and then
    means (context_manager.py:571-576).  Strided input rows (a slice of a longer call)."""
    from infllm_amd import _lib
    lib = _lib.load()
    B, H, n, exc, n_local = 2, 3, 150, 64, 48
    full = _rand((B, H, n + 20, D), 5)
    q = full[:, :, 7:7 + n]
    rope = RopeOracle(D, base=1e4)
    inv_freq = rope.inv_freq.float().cuda()
    qd = full.cuda()[:, :, 7:7 + n]
    qbar = torch.zeros((B, 3, H * D), dtype=torch.float32, device="cuda")
    _lib.check(lib.infllm_chunk_qbar(qd.data_ptr(), qd.stride(0), qd.stride(1), qd.stride(2), B, H, n, exc, inv_freq.data_ptr(),
                                     1.0, n_local - 1, qbar.data_ptr(), torch.cuda.current_stream().cuda_stream), "infllm_chunk_qbar")
    rot = rope.one_angle(q.float(), n_local)
    for j, (a, b) in enumerate(((0, 64), (64, 128), (128, 150))):
        want = rot[:, :, a:b].mean(dim=2).reshape(B, H * D)
        assert torch.allclose(qbar[:, j].cpu(), want, atol=2e-5), float((qbar[:, j].cpu() - want).abs().max())
    assert lib.infllm_chunk_qbar(None, 0, 0, 0, B, H, n, exc, inv_freq.data_ptr(), 1.0, 0, qbar.data_ptr(), None) != 0


# ----------------------------------------------------------------- attention
def _oracle_two_stage(q, stages):
    a = MultiStageOracle(q.shape)
    for i, (k, v, kw) in enumerate(stages):
        a.append(q.float(), k.float(), v.float(), end=(i == len(stages) - 1), get_score=True, **kw)
    return a.get_result()


CASES = [
    # H, Hkv, Lq, Lk, window kwargs
    (4, 1, 64, 192, dict(sliding_window=128)),
    (8, 2, 37, 100, dict(sliding_window=50)),
    (2, 2, 1, 300, dict(sliding_window=256)),
    (3, 3, 130, 130, dict(sliding_window=1000)),
    (4, 2, 96, 257, dict()),
    (4, 1, 50, 200, dict(sliding_window=(170, 64), complement_sliding_window=True)),
    (6, 1, 33, 90, dict(sliding_window=(40, 30))),
    (7, 1, 20, 64, dict(sliding_window=16)),
]


@pytest.mark.parametrize("H,Hkv,Lq,Lk,kw", CASES)
@pytest.mark.parametrize("nsplit", [1, 3])
def test_single_stage_matches_oracle(H, Hkv, Lq, Lk, kw, nsplit):
    ops = _ops()
    B = 2
    q, k, v = _rand((B, H, Lq, D), 10), _rand((B, Hkv, Lk, D), 11), _rand((B, Hkv, Lk, D), 12)
    want, (want_score,) = _oracle_two_stage(q, [(k, v, kw)])
    sw = kw.get("sliding_window")
    if sw is None:
        mask, offset, window = ops.MASK_NONE, 0, 0
    else:
        offset, window = (Lk - Lq, sw) if isinstance(sw, int) else sw
        mask = ops.MASK_COMPLEMENT if kw.get("complement_sliding_window") else ops.MASK_WINDOW
    qd, kd, vd = q.cuda(), k.cuda(), v.cuda()
    o_part = torch.empty((nsplit, B, H, Lq, D), dtype=torch.float16, device="cuda")
    lse_part = torch.empty((nsplit, B, H, Lq), dtype=torch.float32, device="cuda")
    ops.attn_stage_linear(qd, kd, vd, o_part, lse_part, j_lo=0, j_hi=Lk, mask=mask, offset=offset, window=window, nsplit=nsplit)
    out = torch.empty((B, H, Lq, D), dtype=torch.bfloat16, device="cuda")
    lse = torch.empty((B, H, Lq), dtype=torch.float32, device="cuda")
    ops.attn_merge(o_part, lse_part, nsplit, out, lse)
    _check_out(out, want)
    # lse is the base-2 log-sum-exp of the scaled visible logits
    from oracle.multistage import stage_mask, expand_kv
    logits = (q.float() @ expand_kv(k.float(), H).transpose(-1, -2)) / math.sqrt(D)
    vis = stage_mask(Lq, Lk, sw, kw.get("complement_sliding_window", False))
    want_lse = torch.logsumexp(logits.masked_fill(~vis, float("-inf")), dim=-1) / math.log(2.0)
    has = vis.any(dim=-1)
    assert torch.allclose(lse.cpu()[..., has], want_lse[..., has], atol=2e-2)
    assert bool(torch.isinf(lse.cpu()[..., ~has]).all())
    assert float(out.float().cpu()[:, :, ~has].abs().max() if (~has).any() else 0.0) == 0.0
    score = torch.full((B, H, Lk), 7.0, dtype=torch.float32, device="cuda")
    ops.local_score(qd, kd, lse, score, j_lo=0, j_hi=Lk, mask=mask, offset=offset, window=window, accumulate=False)
    assert torch.allclose(score.cpu(), want_score, atol=2e-2, rtol=2e-2), float((score.cpu() - want_score).abs().max())


def test_two_stage_joint_softmax_with_ring_and_pages():
    """Local stage from a wrapped ring + global stage from a page table, as the stream uses them."""
    ops = _ops()
    B, H, Hkv, Lq, n_local, cap = 1, 8, 2, 64, 256, 384
    b0 = 1000                                  # absolute position of the first query
    lo, b1 = b0 - n_local, b0 + Lq
    q = _rand((B, H, Lq, D), 20)
    k_win, v_win = _rand((B, Hkv, b1 - lo, D), 21), _rand((B, Hkv, b1 - lo, D), 22)
    n_glob = 64 * 3 + 50
    k_g, v_g = _rand((B, Hkv, n_glob, D), 23), _rand((B, Hkv, n_glob, D), 24)
    want, (want_ls, _) = _oracle_two_stage(q, [(k_win, v_win, dict(sliding_window=n_local)), (k_g, v_g, dict())])
    ring_k = torch.zeros((B, Hkv, cap, D), dtype=torch.bfloat16, device="cuda")
    ring_v = torch.zeros_like(ring_k)
    rows = torch.arange(lo, b1) % cap
    ring_k[:, :, rows] = k_win.cuda()
    ring_v[:, :, rows] = v_win.cuda()
    qd = q.cuda()
    o_part = torch.empty((2, B, H, Lq, D), dtype=torch.float16, device="cuda")
    lse_part = torch.empty((2, B, H, Lq), dtype=torch.float32, device="cuda")
    ops.attn_stage_linear(qd, ring_k, ring_v, o_part[0:1], lse_part[0:1], cap=cap, j_lo=lo, j_hi=b1,
                          mask=ops.MASK_WINDOW, offset=b0, window=n_local)
    # pages: scattered 64-row tiles inside one pool, the last one partial
    pool_k = torch.zeros((Hkv, 1024, D), dtype=torch.bfloat16, device="cuda")
    pool_v = torch.zeros_like(pool_k)
    starts = [512, 0, 256, 900]
    ent, pos = [], 0
    for s in starts:
        n = min(64, n_glob - pos)
        pool_k[:, s:s + n] = k_g[0, :, pos:pos + n].cuda()
        pool_v[:, s:s + n] = v_g[0, :, pos:pos + n].cuda()
        ent.append((pool_k.data_ptr() + s * D * 2, pool_v.data_ptr() + s * D * 2, 1024 * D, n))
        pos += n
    arr = ops.make_pages(ent)
    import ctypes
    host = torch.empty((len(ent) * 32,), dtype=torch.uint8)
    ctypes.memmove(host.data_ptr(), arr, len(ent) * 32)
    pages = host.cuda()
    ops.attn_stage_paged(qd, pages, len(ent), Hkv, o_part[1:2], lse_part[1:2])
    out = torch.empty((B, H, Lq, D), dtype=torch.bfloat16, device="cuda")
    lse = torch.empty((B, H, Lq), dtype=torch.float32, device="cuda")
    ops.attn_merge(o_part, lse_part, 2, out, lse)
    _check_out(out, want)
    # the same through the one-call forward (both stages + merge), with 2 + 1 key splits: same partial layout rules
    o3 = torch.empty((3, B, H, Lq, D), dtype=torch.float16, device="cuda")
    l3 = torch.empty((3, B, H, Lq), dtype=torch.float32, device="cuda")
    la = ops.linear_stage_args(qd, ring_k, ring_v, o3[0:2], l3[0:2], cap=cap, j_lo=lo, j_hi=b1, mask=ops.MASK_WINDOW,
                               offset=b0, window=n_local, nsplit=2)
    ga = ops.paged_stage_args(qd, pages, len(ent), Hkv, o3[2:3], l3[2:3])
    out2, lse2 = torch.empty_like(out), torch.empty_like(lse)
    ops.attn_fwd(la, ga, out2, lse2)
    _check_out(out2, want)
    # the row sums are taken over bf16-rounded probabilities (what the second MFMA multiplies), so the log-sum-exp
    # depends on how the keys were split at the 2^-9 / sqrt(keys) level
    assert torch.allclose(lse2, lse, atol=1e-3)
    out3 = torch.empty_like(out)
    ops.attn_fwd(None, ga, out3, None)                       # one stage alone
    ops.attn_merge(o_part[1:2], lse_part[1:2], 1, out2, None)
    assert torch.equal(out3, out2)
    from infllm_amd._lib import InfLLMHipError
    with pytest.raises(InfLLMHipError):                      # partial buffers that do not follow one another
        ops.attn_fwd(la, ops.paged_stage_args(qd, pages, len(ent), Hkv, o_part[1:2], lse_part[1:2]), out2, None)
    score = torch.zeros((B, H, cap), dtype=torch.float32, device="cuda")
    ops.local_score(qd, ring_k, lse, score, cap=cap, j_lo=lo, j_hi=b1, mask=ops.MASK_WINDOW, offset=b0, window=n_local,
                    accumulate=True, score_cap=cap)
    ops.local_score(qd, ring_k, lse, score, cap=cap, j_lo=lo, j_hi=b1, mask=ops.MASK_WINDOW, offset=b0, window=n_local,
                    accumulate=True, score_cap=cap)
    assert torch.allclose(score[:, :, rows].cpu(), 2 * want_ls, atol=2e-2, rtol=2e-2)


@pytest.mark.parametrize("Lq,nsplit", [(1, 24), (3, 64), (5, 9)])
def test_decode_shape_many_key_splits(Lq, nsplit):
    """Few query rows and dozens of key splits (what a single-token step launches): the merge of that many
    partials takes its own kernels; output and log-sum-exp against the oracle, lse-only merge against the full one."""
    ops = _ops()
    B, H, Hkv, Lk = 1, 8, 2, 64 * 70
    q, k, v = _rand((B, H, Lq, D), 40), _rand((B, Hkv, Lk, D), 41), _rand((B, Hkv, Lk, D), 42)
    want, _ = _oracle_two_stage(q, [(k, v, dict())])
    qd, kd, vd = q.cuda(), k.cuda(), v.cuda()
    o_part = torch.empty((nsplit, B, H, Lq, D), dtype=torch.float16, device="cuda")
    lse_part = torch.empty((nsplit, B, H, Lq), dtype=torch.float32, device="cuda")
    ops.attn_stage_linear(qd, kd, vd, o_part, lse_part, j_lo=0, j_hi=Lk, nsplit=nsplit)
    out = torch.empty((B, H, Lq, D), dtype=torch.bfloat16, device="cuda")
    lse, lse_only = (torch.empty((B, H, Lq), dtype=torch.float32, device="cuda") for _ in range(2))
    ops.attn_merge(o_part, lse_part, nsplit, out, lse)
    _check_out(out, want)
    logits = torch.einsum("bhqd,bhkd->bhqk", q.float(), k.float().repeat_interleave(H // Hkv, dim=1)) / math.sqrt(D)
    assert torch.allclose(lse.cpu() * math.log(2.0), torch.logsumexp(logits, dim=-1), atol=2e-2)
    from infllm_amd import _lib
    _lib.check(_lib.load().infllm_attn_merge(o_part.data_ptr(), lse_part.data_ptr(), nsplit, B, H, Lq, None, 0, 0, 0,
                                             lse_only.data_ptr(), torch.cuda.current_stream().cuda_stream), "infllm_attn_merge")
    assert torch.allclose(lse_only, lse, atol=1e-5)


def test_operator_class_protocol():
    from infllm_amd.attention.dot_production_attention import get_multi_stage_dot_production_attention
    Attn, flash = get_multi_stage_dot_production_attention(True)
    assert flash is True
    B, H, Hkv, Lq = 1, 4, 2, 48
    q = _rand((B, H, Lq, D), 30)
    k1, v1 = _rand((B, Hkv, 120, D), 31), _rand((B, Hkv, 120, D), 32)
    k2, v2 = _rand((B, Hkv, 70, D), 33), _rand((B, Hkv, 70, D), 34)
    stages = [(k1, v1, dict(sliding_window=64)), (k2, v2, dict(sliding_window=(72, 64), complement_sliding_window=True))]
    want, (ws1, ws2) = _oracle_two_stage(q, stages)
    attn = Attn(q.shape, torch.bfloat16, "cuda")
    attn.append(q.cuda(), k1.cuda(), v1.cuda(), sliding_window=64, get_score=True)
    attn.append(q.cuda(), k2.cuda(), v2.cuda(), sliding_window=(72, 64), complement_sliding_window=True, end=True)
    out, (s1, s2) = attn.get_result()
    _check_out(out, want)
    assert s2 is None and torch.allclose(s1.cpu(), ws1, atol=2e-2, rtol=2e-2)
    with pytest.raises(TypeError):
        Attn(q.shape, torch.float32, "cuda")
    # empty second stage
    attn = Attn(q.shape, torch.bfloat16, "cuda")
    attn.append(q.cuda(), k1.cuda(), v1.cuda(), sliding_window=64)
    attn.append(q.cuda(), k2.cuda()[:, :, :0], v2.cuda()[:, :, :0], end=True)
    want1, _ = _oracle_two_stage(q, [(k1, v1, dict(sliding_window=64))])
    _check_out(attn.get_result()[0], want1)


@pytest.mark.parametrize("Lq,n_local,n_glob,nsplit,H,Hkv", [(64, 256, 64 * 3 + 50, 1, 8, 2), (96, 512, 64 * 9, 4, 8, 2), (33, 100, 40, 3, 4, 4),
                                                        (512, 1024, 64 * 20 + 1, 4, 8, 2), (5, 64, 700, 7, 4, 1)])
def test_both_stages_in_one_launch_equal_the_oracle_and_the_two_launches(Lq, n_local, n_glob, nsplit, H, Hkv):
    """infllm_attn_stages_fused: the ring tiles and the pages as one list divided among the key splits (splits that lie
    in the window, in the pages, or across the seam, where the queries are swapped), against the fp32 oracle and
    against the two-launch form (same joint softmax; the partials are cut elsewhere, so equal to rounding only)."""
    ops = _ops()
    B, cap = 2, (n_local + Lq + 63) // 64 * 64 + 64
    b0 = 5000
    lo, b1 = b0 - n_local, b0 + Lq
    q, qg = _rand((B, H, Lq, D), 60), _rand((B, H, Lq, D), 61)
    k_win, v_win = _rand((B, Hkv, b1 - lo, D), 62), _rand((B, Hkv, b1 - lo, D), 63)
    k_g, v_g = _rand((B, Hkv, n_glob, D), 64), _rand((B, Hkv, n_glob, D), 65)
    ora = MultiStageOracle(q.shape)
    ora.append(q.float(), k_win.float(), v_win.float(), sliding_window=n_local)
    ora.append(qg.float(), k_g.float(), v_g.float(), end=True)
    want, _ = ora.get_result()
    ring_k = torch.zeros((B, Hkv, cap, D), dtype=torch.bfloat16, device="cuda")
    ring_v = torch.zeros_like(ring_k)
    rows = torch.arange(lo, b1) % cap
    ring_k[:, :, rows] = k_win.cuda()
    ring_v[:, :, rows] = v_win.cuda()
    kgd, vgd = k_g.cuda(), v_g.cuda()
    ent = []
    for b in range(B):
        for pos in range(0, n_glob, 64):
            ent.append((kgd[b].data_ptr() + pos * D * 2, vgd[b].data_ptr() + pos * D * 2, n_glob * D, min(64, n_glob - pos)))
    n_pages = len(ent) // B
    arr = ops.make_pages(ent)
    import ctypes
    host = torch.empty((len(ent) * 32,), dtype=torch.uint8)
    ctypes.memmove(host.data_ptr(), arr, len(ent) * 32)
    pages = host.cuda()
    qd, qgd = q.cuda(), qg.cuda()
    o_part = torch.empty((2 * nsplit, B, H, Lq, D), dtype=torch.float16, device="cuda")
    lse_part = torch.empty((2 * nsplit, B, H, Lq), dtype=torch.float32, device="cuda")
    la = ops.linear_stage_args(qd, ring_k, ring_v, o_part[:nsplit], lse_part[:nsplit], cap=cap, j_lo=lo, j_hi=b1, mask=ops.MASK_WINDOW,
                               offset=b0, window=n_local, nsplit=nsplit)
    ga = ops.paged_stage_args(qgd, pages, n_pages, Hkv, o_part[nsplit:], lse_part[nsplit:], nsplit=nsplit)
    two, two_lse = torch.empty((B, H, Lq, D), dtype=torch.bfloat16, device="cuda"), torch.empty((B, H, Lq), device="cuda")
    ops.attn_fwd(la, ga, two, two_lse)
    ops.attn_stages_fused(la, ga)
    one, one_lse = torch.empty_like(two), torch.empty_like(two_lse)
    ops.attn_merge(o_part[:nsplit], lse_part[:nsplit], nsplit, one, one_lse)
    _check_out(one, want)
    assert torch.allclose(one_lse, two_lse, atol=1e-3)
    assert float((one.float() - two.float()).abs().max()) <= 2.0 ** -6 * max(1.0, float(two.float().abs().max()))


# ----------------------------------------------------------------- retrieval
@pytest.mark.parametrize("N,k", [(17, 16), (991, 16), (8192, 16), (5000, 64), (40, 1), (8194, 16), (16384, 64), (20000, 16),
                                 (3000, 1024), (1024, 1024), (2049, 3)])
def test_score_topk_matches_bruteforce(N, k):
    ops = _ops()
    C = 32 * D
    reps = _rand((N, C), 40 + N)
    qbar = torch.randn(C, generator=torch.Generator().manual_seed(41))
    scores = torch.empty((N,), dtype=torch.float32, device="cuda")
    idx = torch.empty((k,), dtype=torch.int32, device="cuda")
    ops.score_topk(reps.cuda(), N, qbar.cuda(), k, scores, idx)
    want = reps.double().numpy() @ qbar.double().numpy()
    got_scores = scores.cpu().double().numpy()
    assert np.allclose(got_scores, want, rtol=1e-4, atol=1e-3)
    got = idx.cpu().tolist()
    assert len(set(got)) == k
    # exactly the top-k of the kernel's own fp32 scores, in descending score like torch.topk (equal scores -> lower index first) ...
    host_scores = scores.cpu().tolist()
    order = sorted(range(N), key=lambda i: (-host_scores[i], i))
    assert got == order[:k]
    # ... and equal to the oracle's set except for candidates within 1e-3 relative of the boundary
    want_set = set(np.argsort(-want, kind="stable")[:k].tolist())
    kth = np.sort(want)[-k]
    for i in set(got) ^ want_set:
        assert abs(want[i] - kth) <= 1e-3 * abs(kth)


@pytest.mark.parametrize("N,k,heads,Q", [(991, 16, 32, 15), (17, 16, 32, 1), (8159, 16, 32, 9), (300, 4, 8, 16), (5000, 64, 4, 3),
                                         (20000, 16, 16, 2)])
def test_several_queries_in_one_pass_give_the_scores_and_ids_of_one_query_at_a_time(N, k, heads, Q):
    """infllm_score_topk_queries against infllm_unit_scores + infllm_topk query by query: the scores bit for bit (a unit's
    score must not depend on which kernel computed it: selections ranked from a call's lists are compared with
    selections over all units), the same ids in the same order."""
    ops = _ops()
    C = heads * D
    reps = _rand((N + 3, C), 60 + N)[:N].cuda()
    qbars = torch.randn((Q, C), generator=torch.Generator().manual_seed(61)).cuda()
    scores = torch.full((Q, N + 5), -7.0, dtype=torch.float32, device="cuda")
    idx = torch.full((Q, k + 2), -1, dtype=torch.int32, device="cuda")
    ops.score_topk_queries(reps, N, qbars, k, scores, idx)
    for q in range(Q):
        one = torch.empty((N,), dtype=torch.float32, device="cuda")
        one_idx = torch.empty((k,), dtype=torch.int32, device="cuda")
        ops.unit_scores(reps, 0, N, qbars[q], one)
        ops.topk(one, N, k, one_idx)
        assert torch.equal(scores[q, :N], one), q
        assert torch.equal(idx[q, :k], one_idx), q
    assert bool((scores[:, N:] == -7.0).all()) and bool((idx[:, k:] == -1).all())      # nothing beyond what was asked for


@pytest.mark.parametrize("n_old,n_new,k,heads", [(991, 4, 16, 32), (40, 1, 16, 32), (16, 16, 16, 8), (300, 7, 4, 16), (5000, 48, 16, 4),
                                                 (64, 3, 1, 32)])
def test_new_units_scored_and_ranked_in_one_launch_equal_the_two_steps(n_old, n_new, k, heads):
    """infllm_score_new_topk against infllm_score_topk over all rows: the new rows' scores bit for bit, the same ids
    (also with exact ties between an old and a new unit, which go to the lower index)."""
    ops = _ops()
    C, N = heads * D, n_old + n_new
    reps = _rand((N, C), 300 + N)
    reps[n_old:n_old + min(2, n_new)] = reps[:min(2, n_new)]              # exact ties old / new
    qbar = torch.randn(C, generator=torch.Generator().manual_seed(43)).cuda()
    repd = reps.cuda()
    want_scores = torch.empty((N,), dtype=torch.float32, device="cuda")
    want_idx = torch.empty((k,), dtype=torch.int32, device="cuda")
    ops.score_topk(repd, N, qbar, k, want_scores, want_idx)
    scores = torch.full((N,), float("nan"), dtype=torch.float32, device="cuda")
    cand = torch.empty((k,), dtype=torch.int32, device="cuda")
    ops.score_topk(repd, n_old, qbar, k, scores, cand)
    idx = torch.empty((k,), dtype=torch.int32, device="cuda")
    ops.score_new_topk(repd, qbar, scores, cand, n_old, n_new, k, idx)
    assert torch.equal(scores, want_scores)
    assert idx.cpu().tolist() == want_idx.cpu().tolist()


def test_topk_with_exact_ties_takes_lowest_indices():
    ops = _ops()
    N, C = 300, 128
    reps = torch.zeros((N, C), dtype=torch.bfloat16)
    reps[:, 0] = 1.0
    reps[200:210, 0] = 2.0
    qbar = torch.zeros(C)
    qbar[0] = 1.0
    scores = torch.empty((N,), dtype=torch.float32, device="cuda")
    idx = torch.empty((16,), dtype=torch.int32, device="cuda")
    ops.score_topk(reps.cuda(), N, qbar.cuda(), 16, scores, idx)
    assert idx.cpu().tolist() == list(range(200, 210)) + [0, 1, 2, 3, 4, 5]
    neg = (-reps).cuda()
    ops.score_topk(neg, N, qbar.cuda(), 4, scores, idx)
    assert idx.cpu().tolist()[:4] == [0, 1, 2, 3]


@pytest.mark.parametrize("N,k,levels", [(6000, 16, 5), (1000, 100, 3), (12000, 300, 40), (70, 70, 2), (16384, 1, 1),
                                        (30000, 50, 7)])
def test_topk_on_heavily_tied_scores_is_the_stable_descending_prefix(N, k, levels):
    """Few distinct score values (negative, zero and positive): the selection must be the first k of a stable
    descending sort, returned in that order, whichever digit pass the search stops in."""
    ops = _ops()
    g = torch.Generator().manual_seed(N + k)
    vals = torch.randint(0, levels, (N,), generator=g).float() - levels // 2
    vals = vals * (1.0 + 2.0 ** -20)                      # differences in the lowest mantissa bits as well
    scores = vals.cuda()
    idx = torch.full((k,), -1, dtype=torch.int32, device="cuda")
    ops.topk(scores, N, k, idx)
    order = sorted(range(N), key=lambda i: (-float(vals[i]), i))
    assert idx.cpu().tolist() == order[:k]


@pytest.mark.parametrize("N,k,pattern", [(6000, 16, "levels"), (16384, 16, "one_group"), (16384, 64, "one_group"), (9000, 16, "falling"),
                                         (9000, 40, "rising"), (8192, 33, "constant"), (700, 64, "levels"), (16, 16, "falling")])
def test_scores_and_selection_in_one_launch_give_the_stable_descending_prefix(N, k, pattern):
    """infllm_score_topk where scoring and selection are ONE launch (rows of 512 elements, k <= 64, N <= 16384), on
    scores made to be exact in fp32 (score = 256 * column 0 + column 1 of small integers): few distinct values, scores
    that fall or rise with the unit number, all equal, and "one_group" - the high scores sit on the units that the
    selection deals to ONE of its thread groups, so its threshold lets more candidates through than it can rank and
    the exact bit-by-bit search takes over.  Always: the first k of a stable descending sort, in that order."""
    ops = _ops()
    g = torch.Generator().manual_seed(N + k)
    n = torch.arange(N)
    if pattern == "levels":
        val = torch.randint(0, 5, (N,), generator=g) - 2
    elif pattern == "falling":
        val = -n
    elif pattern == "rising":
        val = n
    elif pattern == "constant":
        val = torch.full((N,), 7)
    else:
        val = torch.where(n % 512 < 32, 1000 + torch.randint(0, 50, (N,), generator=g), torch.randint(0, 900, (N,), generator=g))
    reps = torch.zeros((N, 512), dtype=torch.bfloat16)
    reps[:, 0] = torch.div(val, 256, rounding_mode="floor").float()
    reps[:, 1] = (val % 256).float()
    qbar = torch.zeros(512)
    qbar[0], qbar[1] = 256.0, 1.0
    scores = torch.full((N,), float("nan"), dtype=torch.float32, device="cuda")
    idx = torch.full((k,), -1, dtype=torch.int32, device="cuda")
    ops.score_topk(reps.cuda(), N, qbar.cuda(), k, scores, idx)
    assert scores.cpu().tolist() == val.float().tolist()
    order = sorted(range(N), key=lambda i: (-int(val[i]), i))
    assert idx.cpu().tolist() == order[:k]
    # the same call again (the launch leaves its ticket slot ready for the next one), and a plain selection for reference
    idx2, idx3 = torch.full_like(idx, -1), torch.full_like(idx, -1)
    ops.score_topk(reps.cuda(), N, qbar.cuda(), k, scores, idx2)
    ops.topk(scores, N, k, idx3)
    assert torch.equal(idx2, idx) and torch.equal(idx3, idx)


@pytest.mark.parametrize("bs,r,H,Hkv", [(128, 4, 32, 8), (8, 2, 4, 2), (100, 1, 3, 3), (64, 64, 2, 1)])
def test_repr_keys_matches_oracle(bs, r, H, Hkv):
    ops = _ops()
    B, cap, n_units, t0 = 2, 640, 3, 600            # units wrap around the end of the ring
    g = torch.Generator().manual_seed(50)
    score = torch.rand((B, H, cap), generator=g)
    ring_k = _rand((B, Hkv, cap, D), 51)
    reps = torch.zeros((B, n_units + 1, H * D), dtype=torch.bfloat16, device="cuda")
    idx = torch.zeros((B, n_units, H, r), dtype=torch.int32, device="cuda")
    ops.repr_keys(score.cuda(), ring_k.cuda(), t0, bs, n_units, r, reps[:, 1], reps.stride(0), reps.stride(1), idx)
    assert float(reps[:, 0].abs().max()) == 0.0
    for b in range(B):
        for u in range(n_units):
            rows = [(t0 + u * bs + i) % cap for i in range(bs)]
            sc = score[b][:, rows]
            want_idx = sc.topk(r, dim=-1).indices
            assert torch.equal(idx[b, u].cpu().long(), want_idx)
            kx = ring_k[b][:, rows].float().repeat_interleave(H // Hkv, dim=0)
            want = torch.gather(kx, 1, want_idx[:, :, None].expand(-1, -1, D)).mean(dim=1).reshape(-1)
            assert torch.allclose(reps[b, u + 1].cpu().float(), want, atol=1e-2, rtol=1e-2)
            assert torch.equal(reps[b, u + 1].cpu(), want.bfloat16())


def test_gather_rows_and_copy_async():
    ops = _ops()
    B, Hkv, cap, bs = 2, 3, 256, 40
    ring = _rand((B, Hkv, cap, D), 60).cuda()
    t0, n_units = 200, 2
    stage = torch.zeros((n_units, B, 2, Hkv, bs, D), dtype=torch.bfloat16, device="cuda")
    ops.gather_rows(ring, t0, n_units * bs, stage[0, 0, 1].data_ptr(), stage.stride(1), stage.stride(3), unit_rows=bs,
                    out_su=stage.stride(0))
    for u in range(n_units):
        rows = [(t0 + u * bs + i) % cap for i in range(bs)]
        assert torch.equal(stage[u, :, 1], ring[:, :, rows])
    assert float(stage[:, :, 0].abs().max()) == 0.0
    host = torch.empty(stage[0].shape, dtype=torch.bfloat16, pin_memory=True)
    ops.copy_async(host, stage[0], stage[0].numel() * 2, 2)
    torch.cuda.synchronize()
    assert torch.equal(host, stage[0].cpu())
    back = torch.zeros_like(stage[0])
    ops.copy_async(back, host, host.numel() * 2, 1)
    torch.cuda.synchronize()
    assert torch.equal(back, stage[0])


def test_fetch_units_reads_pinned_memory_in_one_launch():
    import ctypes
    from infllm_amd import _lib
    lib = _lib.load()
    n, elems = 70, 2 * 3 * 40 * D                    # more units than one launch takes, odd-sized units
    host = torch.empty((n, elems), dtype=torch.bfloat16, pin_memory=True)
    host.copy_(torch.randn(n, elems).bfloat16())
    dev_base = lib.infllm_host_device_pointer(host.data_ptr())
    assert dev_base
    slab = torch.zeros((n + 3, elems), dtype=torch.bfloat16, device="cuda")
    order = torch.randperm(n).tolist()
    src = (ctypes.c_void_p * n)(*[dev_base + i * elems * 2 for i in range(n)])
    dst = (ctypes.c_void_p * n)(*[slab[order[i]].data_ptr() for i in range(n)])
    _lib.check(lib.infllm_fetch_units(src, dst, n, elems * 2, torch.cuda.current_stream().cuda_stream), "fetch")
    torch.cuda.synchronize()
    for i in range(n):
        assert torch.equal(slab[order[i]].cpu(), host[i])
    assert float(slab[n:].abs().max()) == 0.0
    assert lib.infllm_fetch_units(src, dst, 1, 24, None) < 0           # not a multiple of 16 bytes
    assert not lib.infllm_host_device_pointer(None)


def test_bad_arguments_raise():
    ops = _ops()
    from infllm_amd._lib import InfLLMHipError
    q = torch.zeros((1, 4, 8, D), dtype=torch.bfloat16, device="cuda")
    k = torch.zeros((1, 3, 8, D), dtype=torch.bfloat16, device="cuda")
    o = torch.zeros((1, 1, 4, 8, D), dtype=torch.float16, device="cuda")
    l = torch.zeros((1, 1, 4, 8), dtype=torch.float32, device="cuda")
    with pytest.raises(InfLLMHipError):
        ops.attn_stage_linear(q, k, k, o, l)                      # 4 heads over 3 kv heads
    with pytest.raises(InfLLMHipError):
        ops.attn_stage_linear(q, k[:, :1], k[:, :1], o, l, cap=100)   # cap not a multiple of the tile
    with pytest.raises(ValueError):
        ops._bf16_4d(q.float(), "q")
    with pytest.raises(ValueError):
        ops.attn_stage_linear(q, k[:, :1], k[:, :1], o.float(), l)   # partials must be fp16
