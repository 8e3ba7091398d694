"""Torch-tensor wrappers over the C ABI (include/infllm_hip.h).

torch is used for device memory and streams only; every computation below is a
call into libinfllm_hip.so on the current stream.
"""
import math

import torch

from . import _lib
from ._lib import AttnArgs, IngestArgs, Page, ScoreArgs, check

HEAD_DIM = 128
KEY_TILE = 64
MASK_NONE, MASK_WINDOW, MASK_COMPLEMENT = 0, 1, 2
NO_WRAP = 1 << 40          # "cap" of a plain tensor source (a multiple of the key tile)


_pinned_stream = None      # raw hipStream_t fixed by stream_scope(); None -> ask torch every call


def _stream():
    return _pinned_stream if _pinned_stream is not None else torch.cuda.current_stream().cuda_stream


class stream_scope:
    """Pins the launch stream for a run of calls (torch.cuda.current_stream() costs several microseconds)."""

    def __init__(self, raw_stream):
        self.raw = raw_stream

    def __enter__(self):
        global _pinned_stream
        self.prev, _pinned_stream = _pinned_stream, self.raw
        return self

    def __exit__(self, *exc):
        global _pinned_stream
        _pinned_stream = self.prev
        return False


def _need(cond, msg):
    if not cond:
        raise ValueError(msg)


def _bf16_4d(t, name):
    _need(t.is_cuda, f"{name} must be a GPU tensor")
    _need(t.dtype == torch.bfloat16, f"{name} must be bfloat16 (the HIP path computes in bf16), got {t.dtype}")
    _need(t.dim() == 4 and t.shape[-1] == HEAD_DIM, f"{name} must be [B, heads, len, {HEAD_DIM}], got {tuple(t.shape)}")
    if t.stride(-1) != 1 or any(s % 8 for s in t.stride()[:-1]):
        t = t.contiguous()
    return t


def ingest(q, k, v, pos0, glb_pos, inv_freq, distance_scale, ring_k_raw, ring_k_rot, ring_v, ring_score, q_loc, q_glb,
           qpart=None):
    """RoPE + staging of the new tokens; see infllm_ingest."""
    q, k, v = _bf16_4d(q, "q"), _bf16_4d(k, "k"), _bf16_4d(v, "v")
    B, H, n, _ = q.shape
    Hkv = k.shape[1]
    _need(k.shape == v.shape == (B, Hkv, n, HEAD_DIM), "k/v shape mismatch")
    cap = ring_k_raw.shape[2]
    for r in (ring_k_raw, ring_k_rot, ring_v):
        _need(r.is_contiguous() and r.shape == (B, Hkv, cap, HEAD_DIM) and r.dtype == torch.bfloat16, "bad ring")
    _need(ring_score.is_contiguous() and ring_score.shape == (B, H, cap) and ring_score.dtype == torch.float32, "bad score ring")
    for o in (q_loc, q_glb):
        _need(o.is_contiguous() and o.dtype == torch.bfloat16 and o.numel() >= B * H * n * HEAD_DIM, "bad q workspace")
    _need(inv_freq.dtype == torch.float32 and inv_freq.numel() == HEAD_DIM // 2 and inv_freq.is_cuda, "bad inv_freq")
    a = IngestArgs(q.data_ptr(), k.data_ptr(), v.data_ptr(),
                   q.stride(0), q.stride(1), q.stride(2), k.stride(0), k.stride(1), k.stride(2),
                   v.stride(0), v.stride(1), v.stride(2), B, H, Hkv, n, pos0, glb_pos,
                   inv_freq.data_ptr(), float(distance_scale),
                   ring_k_raw.data_ptr(), ring_k_rot.data_ptr(), ring_v.data_ptr(), ring_score.data_ptr(), cap,
                   q_loc.data_ptr(), q_glb.data_ptr(), qpart.data_ptr() if qpart is not None else None)
    check(_lib.load().infllm_ingest(a, _stream()), "infllm_ingest")


def reduce_partials(parts, scale, out):
    """out[b, c] = scale * sum_p parts[b, p, c]."""
    B, n_parts, C = parts.shape
    check(_lib.load().infllm_reduce_partials(parts.data_ptr(), B, n_parts, C, float(scale), out.data_ptr(), _stream()),
          "infllm_reduce_partials")


def rope_rows(x, inv_freq, distance_scale, pos0, consecutive=True):
    """x [B,H,L,128] bf16 (any strides with unit last stride) -> contiguous rows rotated at pos0 + r (or all at pos0)."""
    B, H, L, D = x.shape
    assert x.dtype == torch.bfloat16 and D == 128 and (L == 0 or x.stride(3) == 1)
    out = torch.empty((B, H, L, D), dtype=torch.bfloat16, device=x.device)
    check(_lib.load().infllm_rope_rows(x.data_ptr(), x.stride(0), x.stride(1), x.stride(2), B, H, L, int(pos0),
                                       1 if consecutive else 0, inv_freq.data_ptr(), float(distance_scale), out.data_ptr(),
                                       _stream()), "infllm_rope_rows")
    return out


def block_mean(q_glb, B, H, n, exc, qbar):
    check(_lib.load().infllm_block_mean(q_glb.data_ptr(), B, H, n, exc, qbar.data_ptr(), _stream()), "infllm_block_mean")


def linear_stage_args(q, k, v, o_part, lse_part, *, cap=None, j_lo=0, j_hi=None, mask=MASK_NONE, offset=0, window=0,
                      nsplit=1, softmax_scale=None):
    """Argument block of one stage over a linear key source.  q [B,H,Lq,D]; k/v [B,Hkv,rows,D] (rows = ring rows)."""
    B, H, Lq, D = q.shape
    Hkv = k.shape[1]
    if cap is None:
        cap = NO_WRAP
    if j_hi is None:
        j_hi = k.shape[2]
    _need(o_part.dtype == torch.float16 and lse_part.dtype == torch.float32, "partials are fp16 rows with fp32 log-sum-exps")
    a = AttnArgs()
    a.d_q, a.q_sb, a.q_sh, a.q_sl = q.data_ptr(), q.stride(0), q.stride(1), q.stride(2)
    a.B, a.H, a.Hkv, a.Lq = B, H, Hkv, Lq
    a.d_k, a.d_v = k.data_ptr(), v.data_ptr()
    a.k_sb, a.k_sh, a.k_sl = k.stride(0), k.stride(1), k.stride(2)
    a.v_sb, a.v_sh, a.v_sl = v.stride(0), v.stride(1), v.stride(2)
    a.cap, a.j_lo, a.j_hi = cap, j_lo, j_hi
    a.mask, a.offset, a.window = mask, offset, window
    a.d_pages, a.n_pages, a.nsplit = None, 0, nsplit
    a.softmax_scale = softmax_scale if softmax_scale is not None else 1.0 / math.sqrt(D)
    a.d_o_part, a.d_lse_part = o_part.data_ptr(), lse_part.data_ptr()
    return a


def paged_stage_args(q, pages_dev, n_pages, Hkv, o_part, lse_part, *, nsplit=1, softmax_scale=None):
    """Argument block of one stage over a device page table [B, n_pages] of infllm_page entries."""
    B, H, Lq, D = q.shape
    _need(o_part.dtype == torch.float16 and lse_part.dtype == torch.float32, "partials are fp16 rows with fp32 log-sum-exps")
    a = AttnArgs()
    a.d_q, a.q_sb, a.q_sh, a.q_sl = q.data_ptr(), q.stride(0), q.stride(1), q.stride(2)
    a.B, a.H, a.Hkv, a.Lq = B, H, Hkv, Lq
    a.d_pages, a.n_pages, a.nsplit = pages_dev.data_ptr(), n_pages, nsplit
    a.cap = KEY_TILE
    a.softmax_scale = softmax_scale if softmax_scale is not None else 1.0 / math.sqrt(D)
    a.d_o_part, a.d_lse_part = o_part.data_ptr(), lse_part.data_ptr()
    return a


def attn_stage_linear(q, k, v, o_part, lse_part, **kw):
    """One stage over a linear key source (see linear_stage_args)."""
    check(_lib.load().infllm_attn_stage(linear_stage_args(q, k, v, o_part, lse_part, **kw), _stream()), "infllm_attn_stage")


def attn_stage_paged(q, pages_dev, n_pages, Hkv, o_part, lse_part, **kw):
    """One stage over a device page table (see paged_stage_args)."""
    check(_lib.load().infllm_attn_stage(paged_stage_args(q, pages_dev, n_pages, Hkv, o_part, lse_part, **kw), _stream()),
          "infllm_attn_stage")


def attn_fwd(local_args, global_args, out, lse):
    """Both stages (either may be None) and their merge in one call; out bf16 [B,H,Lq,D], lse fp32 [B,H,Lq] or None."""
    _need(out.stride(-1) == 1 and out.dtype == torch.bfloat16, "bad merge output")
    check(_lib.load().infllm_attn_fwd(local_args, global_args, out.data_ptr(), out.stride(0), out.stride(1), out.stride(2),
                                      lse.data_ptr() if lse is not None else None, _stream()), "infllm_attn_fwd")


def attn_stages_fused(local_args, global_args):
    """Both stages in one launch: one list of tiles, local_args.nsplit partials at local_args' partial buffers."""
    check(_lib.load().infllm_attn_stages_fused(local_args, global_args, _stream()), "infllm_attn_stages_fused")


NOALLOC_MAX_PART_ROWS = 65536       # INFLLM_NOALLOC_MAX_PART_ROWS


def attn_fwd_noalloc(local_args, global_args, out, lse):
    """attn_fwd with the partial rows in the library's built-in scratch array (the argument blocks' o_part / lse_part
    are ignored); allocates nothing.  Calls on one GPU must not overlap."""
    _need(out.stride(-1) == 1 and out.dtype == torch.bfloat16, "bad merge output")
    check(_lib.load().infllm_attn_fwd_noalloc(local_args, global_args, out.data_ptr(), out.stride(0), out.stride(1), out.stride(2),
                                              lse.data_ptr() if lse is not None else None, _stream()), "infllm_attn_fwd_noalloc")


def attn_merge(o_part, lse_part, P, out, lse):
    """Join P partials: out bf16 [B,H,Lq,D] (any strides with contiguous rows), lse fp32 [B,H,Lq]."""
    B, H, Lq, D = out.shape
    _need(out.stride(-1) == 1 and out.dtype == torch.bfloat16, "bad merge output")
    _need(o_part.dtype == torch.float16, "partials are fp16 rows")
    check(_lib.load().infllm_attn_merge(o_part.data_ptr(), lse_part.data_ptr(), P, B, H, Lq,
                                        out.data_ptr(), out.stride(0), out.stride(1), out.stride(2),
                                        lse.data_ptr() if lse is not None else None, _stream()), "infllm_attn_merge")


def local_score(q, k, lse, score, *, cap=None, j_lo=0, j_hi=None, mask=MASK_NONE, offset=0, window=0,
                accumulate=True, score_cap=None, softmax_scale=None):
    """score[b,h,j % score_cap] (+)= column sums of the stage's final probabilities."""
    B, H, Lq, D = q.shape
    a = ScoreArgs()
    a.d_q, a.q_sb, a.q_sh, a.q_sl = q.data_ptr(), q.stride(0), q.stride(1), q.stride(2)
    a.B, a.H, a.Hkv, a.Lq = B, H, k.shape[1], Lq
    a.d_k, a.k_sb, a.k_sh, a.k_sl = k.data_ptr(), k.stride(0), k.stride(1), k.stride(2)
    a.cap = cap if cap is not None else NO_WRAP
    a.j_lo, a.j_hi = j_lo, (j_hi if j_hi is not None else k.shape[2])
    a.mask, a.accumulate, a.offset, a.window = mask, int(accumulate), offset, window
    a.d_lse = lse.data_ptr()
    a.softmax_scale = softmax_scale if softmax_scale is not None else 1.0 / math.sqrt(D)
    a.d_score, a.score_sb, a.score_sh = score.data_ptr(), score.stride(0), score.stride(1)
    a.score_cap = score_cap if score_cap is not None else NO_WRAP
    check(_lib.load().infllm_local_score(a, _stream()), "infllm_local_score")


def score_topk(reps, n, qbar, k, scores, idx):
    """scores[:n] = reps[:n] @ qbar; idx[:k] = indices of the k largest, descending score."""
    check(_lib.load().infllm_score_topk(reps.data_ptr(), reps.stride(0), n, reps.shape[1], qbar.data_ptr(), k,
                                        scores.data_ptr(), idx.data_ptr() if idx is not None else None, _stream()),
          "infllm_score_topk")


def unit_scores(reps, first, count, qbar, scores):
    """scores[first:first+count] = reps[first:first+count] @ qbar."""
    check(_lib.load().infllm_unit_scores(reps.data_ptr(), reps.stride(0), first, count, reps.shape[1], qbar.data_ptr(),
                                         scores.data_ptr(), _stream()), "infllm_unit_scores")


def score_topk_queries(reps, n, qbars, k, scores, idx):
    """scores[q, :n] = reps[:n] @ qbars[q] and idx[q, :k] = indices of the k largest, descending score, for every query q
    in one pass over the representatives."""
    rc = _lib.load().infllm_score_topk_queries(reps.data_ptr(), reps.stride(0), n, reps.shape[1], qbars.data_ptr(), qbars.stride(0),
                                               qbars.shape[0], k, scores.data_ptr(), scores.stride(0), idx.data_ptr(), idx.stride(0),
                                               _stream())
    if rc == 1:
        raise ValueError(f"score_topk_queries: rows of {reps.shape[1]} elements (supported: 512, 1024, 2048, 4096)")
    check(rc, "infllm_score_topk_queries")


def score_new_topk(reps, qbar, scores, cand, first_new, n_new, k, idx):
    """scores[first_new:first_new+n_new] = reps[those rows] @ qbar, then idx[:k] = the top-k over all first_new + n_new
    scores, given cand = the top-k of the first first_new."""
    check(_lib.load().infllm_score_new_topk(reps.data_ptr(), reps.stride(0), reps.shape[1], qbar.data_ptr(), scores.data_ptr(),
                                            cand.data_ptr(), cand.numel(), first_new, n_new, k, idx.data_ptr(), _stream()),
          "infllm_score_new_topk")


def topk(scores, n, k, idx):
    """idx[:k] = indices of the k largest of scores[:n] in descending score (lower index first among equal scores)."""
    check(_lib.load().infllm_topk(scores.data_ptr(), n, k, idx.data_ptr(), _stream()), "infllm_topk")


def repr_keys(ring_score, ring_k_raw, t0, bs, n_units, repr_topk, rep_out, rep_sb, rep_su, idx_out=None):
    B, H, cap = ring_score.shape
    Hkv = ring_k_raw.shape[1]
    check(_lib.load().infllm_repr_keys(ring_score.data_ptr(), ring_k_raw.data_ptr(), cap, B, H, Hkv, t0, bs, n_units,
                                       repr_topk, rep_out.data_ptr(), rep_sb, rep_su,
                                       idx_out.data_ptr() if idx_out is not None else None, _stream()), "infllm_repr_keys")


def gather_rows(ring, t0, n, out_ptr, out_sb, out_sh, unit_rows=None, out_su=0):
    """Ring rows (t0+r) % cap, r < n, of every kv head -> out_ptr + b*out_sb + (r//unit_rows)*out_su + h*out_sh + (r%unit_rows)*D."""
    B, Hkv, cap, _ = ring.shape
    check(_lib.load().infllm_gather_rows(ring.data_ptr(), cap, B, Hkv, t0, n, unit_rows if unit_rows else max(n, 1),
                                         out_ptr, out_sb, out_su, out_sh, _stream()), "infllm_gather_rows")


def copy_async(dst, src, nbytes, kind, stream=None):
    """kind: 1 host->device, 2 device->host, 3 device->device (raw addresses or tensors)."""
    d = dst.data_ptr() if torch.is_tensor(dst) else dst
    s = src.data_ptr() if torch.is_tensor(src) else src
    check(_lib.load().infllm_copy_async(d, s, nbytes, kind, stream if stream is not None else _stream()), "infllm_copy_async")


def make_pages(entries):
    """entries: list of (k_addr, v_addr, head_stride, n_valid) -> ctypes array of infllm_page."""
    arr = (Page * max(len(entries), 1))()
    for i, (k, v, hs, n) in enumerate(entries):
        arr[i].k, arr[i].v, arr[i].head_stride, arr[i].n_valid = k, v, hs, n
    return arr
