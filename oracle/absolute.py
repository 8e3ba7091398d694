"""Oracle, second derivation: the path in absolute stream positions (test infrastructure only).

``oracle.stream`` follows the reference's window-relative cursors.  This module
re-derives what every execution block sees directly from token positions in the
whole stream, with closed forms instead of cursors, so that the two can be
checked against each other (a slip in one's index arithmetic fails the
comparison).  It is a brute force: the full stream is held and every block is
recomputed from it.  fp64 throughout, complex-number RoPE.

For a block of queries at positions [b0, b1) (b0 = tokens consumed before it):

  init_len(e) = min(n_init, max(e - n_local, 0))            evaluated at e = b0
  n_units(e)  = max(0, (e - n_init - n_local) // block_size)
  unit u      = tokens [n_init + u*bs, n_init + (u+1)*bs)
  cursor(e)   = init_len(e) + n_units(e) * bs                 first un-carved token

  local stage : keys kp in [max(b0 - n_local, 0), b1), visible to query qp iff
                0 <= qp - kp < n_local; logit from RoPE at relative distance qp - kp
                (context_manager.py:480-489, 772-773; rope.py:107-112)
  global stage: tokens of the retrieved units, tokens [0, init_len(b0)) and the
                overflow tokens [cursor(b0), b1 - n_local); every one of them is
                visible to every query of the block at the fixed relative distance
                n_local - 1 (context_manager.py:386-451, 744-747).  Overflow tokens
                that are still inside an early query's local window are therefore
                counted twice for that query, as in the reference.
  one softmax over both stages (torch_impl.py:15-36).

Token scores: score[h, t] += sum over the block's queries of the local-stage
probability of key t (context_manager.py:623-625).  When n_units grows at a
block end, the new unit's representative is the mean of its repr_topk
highest-scored keys per query head (context_manager.py:268-277, 664-670), and
retrieval is the top-k of <representative, mean global query of the block>
(:366-383) once there are more than topk units.
"""
import math
import torch


def _rot_complex(x, pos, inv_freq):
    """Rotate x[..., L, D] (half-split pairing) by angle pos[l] * inv_freq[i], in fp64."""
    half = x.shape[-1] // 2
    z = torch.complex(x[..., :half], x[..., half:])
    ang = pos.to(torch.float64)[:, None] * inv_freq[None, :]
    z = z * torch.polar(torch.ones_like(ang), ang)
    return torch.cat((z.real, z.imag), dim=-1)


def block_boundaries(call_lengths, exc):
    """Execution-block [b0, b1) spans for a stream fed in calls of the given lengths."""
    spans, pos = [], 0
    for L in call_lengths:
        for st in range(0, L, exc):
            ed = min(st + exc, L)
            spans.append((pos + st, pos + ed))
        pos += L
    return spans


def run_absolute(q, k, v, call_lengths, n_init, n_local, block_size, topk, exc_block_size,
                 repr_topk=1, base=10000, distance_scale=1.0, forced_topk=None, forced_repr=None):
    """q [H,T,D], k/v [Hkv,T,D] (one batch row).  Returns dict(out[H,T,D], selected, reps, score)."""
    q, k, v = q.double(), k.double(), v.double()
    H, T, D = q.shape
    G = H // k.shape[0]
    kx, vx = k.repeat_interleave(G, dim=0), v.repeat_interleave(G, dim=0)
    inv_freq = (1.0 / (base ** (torch.arange(0, D, 2, dtype=torch.float64) / D))) * distance_scale
    out = torch.zeros(H, T, D, dtype=torch.float64)
    score = torch.zeros(H, T, dtype=torch.float64)
    reps, selected_log, unit_scores_log = [], [], []

    init_len = lambda e: min(n_init, max(e - n_local, 0))
    n_units = lambda e: max(0, (e - n_init - n_local) // block_size)
    fixed = torch.tensor([n_local - 1])

    for bi, (b0, b1) in enumerate(block_boundaries(call_lengths, exc_block_size)):
        nq = b1 - b0
        qpos = torch.arange(b0, b1)
        # ---- local stage
        lo = max(b0 - n_local, 0)
        kpos = torch.arange(lo, b1)
        ql = _rot_complex(q[:, b0:b1], qpos - lo, inv_freq)
        kl = _rot_complex(kx[:, lo:b1], kpos - lo, inv_freq)
        dist = qpos[:, None] - kpos[None, :]
        vis = (dist >= 0) & (dist < n_local)
        s_loc = (ql @ kl.transpose(-1, -2)).masked_fill(~vis, float("-inf"))
        # ---- retrieval
        N = n_units(b0)
        qg = _rot_complex(q[:, b0:b1], fixed.expand(nq), inv_freq)
        if N <= topk:
            sel, us = list(range(N)), None
        else:
            us = torch.stack(reps[:N]) @ qg.mean(dim=1).reshape(H * D)
            sel = sorted(us.topk(topk).indices.tolist())
            if forced_topk is not None and forced_topk[bi] is not None:
                sel = sorted(forced_topk[bi])
        selected_log.append(sel)
        unit_scores_log.append(us)
        # ---- global stage token set (absolute positions)
        toks = []
        for u in sel:
            toks.extend(range(n_init + u * block_size, n_init + (u + 1) * block_size))
        toks.extend(range(0, init_len(b0)))
        toks.extend(range(init_len(b0) + N * block_size, max(b1 - n_local, init_len(b0) + N * block_size)))
        toks = torch.tensor(toks, dtype=torch.int64)
        s_glb = qg @ kx[:, toks].transpose(-1, -2)
        # ---- joint softmax
        p = torch.softmax(torch.cat((s_loc, s_glb), dim=-1) / math.sqrt(D), dim=-1)
        p_loc, p_glb = p[..., :kpos.numel()], p[..., kpos.numel():]
        out[:, b0:b1] = p_loc @ vx[:, lo:b1] + p_glb @ vx[:, toks]
        score[:, lo:b1] += p_loc.sum(dim=-2)
        # ---- units carved at this block end
        for u in range(N, n_units(b1)):
            t0 = n_init + u * block_size
            sc = score[:, t0:t0 + block_size]
            idx = sc.topk(repr_topk, dim=-1).indices
            if forced_repr is not None and forced_repr[u] is not None:
                idx = torch.as_tensor(forced_repr[u], dtype=torch.int64)
            rows = torch.gather(kx[:, t0:t0 + block_size], 1, idx[:, :, None].expand(-1, -1, D))
            reps.append(rows.mean(dim=1).reshape(H * D))
    return dict(out=out, selected=selected_log, unit_scores=unit_scores_log, reps=reps, score=score)
