"""Oracle: the streaming memory state machine (test infrastructure only).

A CPU restatement, in fp32 torch, of ``ContextManager``
(inf_llm/attention/context_manager.py:196-816).  Like the reference it keeps
window-relative state: the local window, the "remainder" (tokens that have not
been carved into memory units yet, a superset of the window) with a pair of
cursors into it, the attention-sink ("init") tokens, the carved units with one
representative vector each, and a model of the GPU unit cache.

Per append() call (context_manager.py:682-813):
  1. new k/v join the local window and the remainder; the score track gets
     zeros for them (:719-741);
  2. the "global" query is the query rotated to the single position n_local-1
     (:744-747);
  3. for every execution block of at most exc_block_size queries (:762-791):
       a. local stage: queries x window slice, window-relative RoPE, causal
          sliding-window mask, probability column sums requested (:480-489);
       b. retrieval: all units while there are <= topk of them, otherwise the
          top-k of <representative, mean global query> (:366-383, 159-163);
       c. unit-cache bookkeeping (:495-515, 246-265) - residency only;
       d. global stage keys: selected units, init tokens, overflow remainder
          (:386-451); its complement-window mask is passed with the offset of
          :437, which makes every key visible to every query of the block;
       e. one softmax over both stages (torch_impl.py:15-36);
       f. score accumulation, init peeling and unit carving (:614-679);
  4. window / remainder trimming (:796-806).

Two hooks let a test follow another implementation's discrete choices where
the acceptance rule allows them to differ (near-ties): ``topk_hook`` and
``repr_hook``.  They receive the oracle's own fp32 scores and may return the
choice to adopt, or None to keep the oracle's.  A selection is an ORDERED list,
in the order torch.topk returns it (descending score, :163): the residency
policy inserts a block's missed units in that order (:495-515), and the order
breaks ties between equal stamps at later evictions (:253-265).

``rep_dtype`` rounds every representative to that dtype when it is stored: the
reference keeps them in a VectorTensor of the model dtype (:321-328, 675), so
torch.bfloat16 restates its bf16 runs; None keeps the compute dtype.

``q_dtype`` restates the roundings the reference's low-precision runs apply on the way
to the mean query of a block: the one-angle-rotated queries are a tensor of the model
dtype and so is their mean (context_manager.py:373-375), i.e. every rotated query is
rounded before the sum and the mean after it.  None keeps the compute dtype throughout
(the HIP path sums the unrounded fp32 rotations and keeps the mean in fp32).

``StreamOracle.from_state`` starts from a snapshot (window, un-carved tail with
its score track, init tokens, units, representatives - the fields of
context_manager.py:309-363 restated in absolute terms) instead of an empty
stream, so that a few execution blocks at the end of a stream too long for the
CPU can be recomputed.
"""
import torch

from .multistage import MultiStageOracle


class UnitCacheModel:
    """Residency model of the GPU unit cache (context_manager.py:6-26, 246-265, 495-515).

    ``cached`` maps unit id -> value in insertion order, exactly like the
    reference's dict: eviction candidates are visited in ascending value, ties
    in dict order (stable sort), selected units are skipped.
    """

    def __init__(self, capacity, strategy="lru", score_decay=None):
        if strategy not in ("lru", "lru-s", "fifo"):
            raise AssertionError(strategy)
        self.capacity = capacity
        self.strategy = strategy
        self.score_decay = score_decay
        self.cached = {}
        self.clock = 0
        self.events = []         # per block: dict(selected, misses, evicted)

    def touch(self, selected):
        selected = list(selected)
        misses = [b for b in selected if b not in self.cached]
        surplus = len(self.cached) - self.capacity + len(misses)
        evicted = []
        if surplus > 0:
            for unit, _ in sorted(self.cached.items(), key=lambda kv: kv[1]):
                if unit not in selected:
                    evicted.append(unit)
                if len(evicted) >= surplus:
                    break
            for unit in evicted:
                del self.cached[unit]
        if self.strategy == "lru":
            self.clock += 1
            for b in selected:
                self.cached[b] = self.clock
        elif self.strategy == "fifo":
            # not in the reference (README.md:83-84 names it, the code asserts
            # lru / lru-s only): a unit keeps the stamp of its first load.
            self.clock += 1
            for b in selected:
                self.cached.setdefault(b, self.clock)
        else:
            for b in selected:
                self.cached[b] = 0
        assert len(self.cached) <= self.capacity, "unit cache overflow (topk > max_cached_block)"
        self.events.append(dict(selected=sorted(selected), order=list(selected), misses=sorted(misses), evicted=evicted))

    def add_scores(self, units, unit_scores):
        """lru-s (context_manager.py:454-470): decay every value, add the block's mass."""
        for u in self.cached:
            self.cached[u] = self.cached[u] * self.score_decay
        for u, s in zip(units, unit_scores):
            self.cached[u] += s


class StreamOracle:
    def __init__(self, rope, n_init, n_local, block_size, max_cached_block, topk,
                 exc_block_size, score_decay=None, repr_topk=1, cache_strategy="lru",
                 perhead=False, topk_hook=None, repr_hook=None, chunk_topk_calc=None, rep_dtype=None, q_dtype=None):
        assert exc_block_size <= n_local                      # context_manager.py:219
        self.chunk_topk_calc = chunk_topk_calc
        self.rope = rope
        self.n_init, self.n_local = n_init, n_local
        self.block_size, self.topk = block_size, topk
        self.exc_block_size = exc_block_size
        self.repr_topk = repr_topk
        self.max_cached_block = max_cached_block
        self.cache_strategy = cache_strategy
        self.score_decay = score_decay
        self.perhead = perhead
        self.topk_hook, self.repr_hook = topk_hook, repr_hook
        self.rep_dtype = rep_dtype
        self.q_dtype = q_dtype
        self.length = 0
        self.ready = False
        self._chunk_plan = None
        self.block_trace = []     # one dict per execution block
        self.unit_trace = []      # one dict per carved unit

    # ------------------------------------------------------------------ state
    def _setup(self, q, k):
        self.B, self.H, _, self.D = q.shape
        self.Hkv = k.shape[1]
        z = lambda h: torch.zeros(self.B, h, 0, self.D, dtype=q.dtype)
        self.win_k, self.win_v = z(self.Hkv), z(self.Hkv)
        self.rem_k, self.rem_v = z(self.Hkv), z(self.Hkv)
        self.rem_score = torch.zeros(self.B, self.H, 0, dtype=q.dtype)
        self.init_k, self.init_v = z(self.Hkv), z(self.Hkv)
        self.init_full = False
        self.units = [[] for _ in range(self.B)]          # (k, v) each [Hkv, bs, D]
        self.reps = [[] for _ in range(self.B)]           # [H*D] each
        self.n_units = 0
        self.cache = [UnitCacheModel(self.max_cached_block, self.cache_strategy, self.score_decay)
                      for _ in range(self.B)]
        self.ready = True

    def size(self):
        return self.length

    def from_state(self, state, dtype=torch.float32):
        """Continue a stream from a snapshot.  ``state``: length T; tail_k / tail_v [B,Hkv,T-cursor,D], the tokens
        not carved yet (context_manager.py:333-336: the remainder, whose last n_local tokens are the local window,
        :330-331); tail_score [B,H,T-cursor] or None (:338); init_k / init_v [B,Hkv,init_len,D] (:341-343); units:
        anything indexable by unit id that yields [B,2,Hkv,bs,D] (K at index 0, V at 1; :317, 652-662), with n_units
        entries; reps [B,n_units,H*D] (:321-328).  The counts must satisfy the closed forms of :614-679.  The unit
        cache starts empty.  Unit tensors are kept as they are given and converted when a block reads them."""
        assert not self.ready and self.length == 0
        f = lambda t: t.detach().to("cpu").to(dtype)
        tail_k, tail_v = f(state["tail_k"]), f(state["tail_v"])
        T = int(state["length"])
        self.B, self.Hkv, n_tail, self.D = tail_k.shape
        reps = state.get("reps")
        self.H = reps.shape[2] // self.D if reps is not None and reps.numel() else int(state["num_heads"])
        init_len = min(self.n_init, max(T - self.n_local, 0))
        n_units = max(0, (T - self.n_init - self.n_local) // self.block_size)
        assert n_tail == T - init_len - n_units * self.block_size, (n_tail, T, init_len, n_units)
        self.win_k, self.win_v = tail_k[:, :, -self.n_local:], tail_v[:, :, -self.n_local:]
        self.rem_k, self.rem_v = tail_k, tail_v
        sc = state.get("tail_score")
        self.rem_score = f(sc) if sc is not None else torch.zeros(self.B, self.H, n_tail, dtype=dtype)
        assert self.rem_score.shape == (self.B, self.H, n_tail)
        self.init_k, self.init_v = f(state["init_k"]), f(state["init_v"])
        assert self.init_k.shape[2] == init_len
        self.init_full = init_len == self.n_init
        units = state.get("units")
        self.units = [[(units[i][u, 0], units[i][u, 1]) for i in range(n_units)] for u in range(self.B)]
        reps_f = f(reps[:, :n_units]) if n_units else None
        self.reps = [[reps_f[u, i] for i in range(n_units)] for u in range(self.B)]
        self.n_units = n_units
        self.cache = [UnitCacheModel(self.max_cached_block, self.cache_strategy, self.score_decay) for _ in range(self.B)]
        self.length = T
        self.ready = True
        return self

    def _group(self, x):
        """[B, Hkv, L, D] -> [B, H, L, D] (context_manager.py:280-289)."""
        if self.H == self.Hkv:
            return x
        return x.repeat_interleave(self.H // self.Hkv, dim=1)

    # -------------------------------------------------------------- retrieval
    def _retrieve_chunk(self, gq_chunk):
        """context_manager.py:548-612: the selections of every execution block of a chunk, all against the
        units that exist when the chunk starts.  The score is the head MEAN of q-bar_h . rep_h (a positive
        multiple of the per-block score of :159-163, so the same ranking)."""
        n_blocks = -(-gq_chunk.shape[2] // self.exc_block_size)
        out = []
        for j in range(n_blocks):
            blk = gq_chunk[:, :, j * self.exc_block_size:(j + 1) * self.exc_block_size]
            if self.n_units <= self.topk:
                out.append(([list(range(self.n_units)) for _ in range(self.B)], [None] * self.B))
                continue
            mean_q = blk.mean(dim=2)                                           # [B, H, D]
            chosen, scores = [], []
            for u in range(self.B):
                reps = torch.stack(self.reps[u]).reshape(self.n_units, self.H, self.D)
                sc = torch.einsum("nhd,hd->nh", reps, mean_q[u]).mean(dim=1)
                pick = sc.topk(self.topk).indices.tolist()                     # descending score, as :586 / :604 return it
                if self.topk_hook is not None:
                    other = self.topk_hook(len(self.block_trace) + j, u, sc * self.H)
                    if other is not None:
                        pick = list(other)
                chosen.append(pick)
                scores.append(sc * self.H)
            out.append((chosen, scores))
        return out

    def _retrieve(self, gq_block):
        if self._chunk_plan is not None:                                       # :366-383, the cached branch
            return self._chunk_plan[self._chunk_pos]
        if self.n_units <= self.topk:
            chosen = [list(range(self.n_units)) for _ in range(self.B)]
            scores = [None] * self.B
        else:
            if self.q_dtype is not None:                                       # :373-375 in the model dtype
                mean_q = gq_block.to(self.q_dtype).float().mean(dim=2).to(self.q_dtype).to(gq_block.dtype)
            else:
                mean_q = gq_block.mean(dim=2)
            mean_q = mean_q.reshape(self.B, self.H * self.D)
            chosen, scores = [], []
            for u in range(self.B):
                reps = torch.stack(self.reps[u])                       # [N, H*D]
                s = reps @ mean_q[u]
                pick = s.topk(self.topk).indices.tolist()                      # descending score (:163)
                if self.topk_hook is not None:
                    other = self.topk_hook(len(self.block_trace), u, s)
                    if other is not None:
                        pick = list(other)
                chosen.append(pick)
                scores.append(s)
        return chosen, scores

    def _representative(self, u, unit_k, unit_score):
        """context_manager.py:268-277, 664-670 for one batch row: [Hkv,bs,D],[H,bs] -> [H*D]."""
        idx = unit_score.topk(self.repr_topk, dim=-1).indices                 # [H, r]
        if self.repr_hook is not None:
            other = self.repr_hook(len(self.units[u]), u, unit_score)
            if other is not None:
                idx = torch.as_tensor(other, dtype=torch.int64)
        k_full = self._group(unit_k[None])[0]                                  # [H, bs, D]
        rows = torch.gather(k_full, 1, idx[:, :, None].expand(-1, -1, self.D))
        rep = rows.mean(dim=1).reshape(self.H * self.D)
        if self.rep_dtype is not None:
            rep = rep.to(self.rep_dtype).to(rows.dtype)
        return rep, idx

    # ------------------------------------------------------------- one block
    def _block(self, q, win_k, win_v, gq, cur_st, cur_ed):
        len_q = q.shape[-2]
        q_rot, k_rot = self.rope.window(q, win_k)
        attn = MultiStageOracle(q.shape, q.dtype)
        attn.append(q_rot, k_rot, win_v, sliding_window=self.n_local, get_score=True)

        chosen, unit_scores = self._retrieve(gq)
        for u in range(self.B):
            self.cache[u].touch(chosen[u])

        overflow = max(cur_ed - cur_st + len_q - self.n_local, 0)
        parts_k, parts_v = [], []
        for u in range(self.B):
            as_mine = lambda t: t.to(device=q.device, dtype=q.dtype)               # units given to from_state stay as they came
            ks = [as_mine(self.units[u][b][0]) for b in sorted(chosen[u])]         # :399 sorts before placing the units
            vs = [as_mine(self.units[u][b][1]) for b in sorted(chosen[u])]
            ks += [self.init_k[u], self.rem_k[u, :, cur_st:cur_st + overflow]]
            vs += [self.init_v[u], self.rem_v[u, :, cur_st:cur_st + overflow]]
            parts_k.append(torch.cat(ks, dim=-2))
            parts_v.append(torch.cat(vs, dim=-2))
        glob_k, glob_v = torch.stack(parts_k), torch.stack(parts_v)
        n_unit_keys = len(chosen[0]) * self.block_size
        mask_offset = self.rem_k.shape[-2] + n_unit_keys + self.init_k.shape[-2]   # :437
        want_glob_score = self.cache_strategy == "lru-s"
        attn.append(gq, glob_k, glob_v, end=True, get_score=want_glob_score,
                    sliding_window=(mask_offset, self.n_local), complement_sliding_window=True)
        out, (loc_score, glob_score) = attn.get_result()

        if want_glob_score:
            per_unit = glob_score[:, :, :n_unit_keys].reshape(self.B, self.H, len(chosen[0]), self.block_size)
            per_unit = per_unit.sum(dim=-1).sum(dim=1)
            for u in range(self.B):
                self.cache[u].add_scores(sorted(chosen[u]), per_unit[u].tolist())

        self.block_trace.append(dict(
            selected=[sorted(c) for c in chosen], order=[list(c) for c in chosen], unit_scores=unit_scores, n_units=self.n_units,
            init_len=self.init_k.shape[-2], overflow=overflow, global_len=glob_k.shape[-2],
            local_len=win_k.shape[-2]))
        return out, loc_score

    def _after_block(self, n_new, win_len, loc_score, cur_st, cur_ed):
        """context_manager.py:614-679."""
        ed = cur_ed + n_new
        st = cur_st
        assert loc_score.shape == (self.B, self.H, win_len)                    # :623
        loc_score = loc_score[:, :, -n_new - self.n_local:]                    # :624 (the whole of it)
        self.rem_score[:, :, ed - loc_score.shape[-1]:ed] += loc_score
        live = ed - st
        if not self.init_full and live > self.n_local:
            take = min(self.n_init - self.init_k.shape[-2], live - self.n_local)
            self.init_k = torch.cat((self.init_k, self.rem_k[:, :, st:st + take]), dim=-2)
            self.init_v = torch.cat((self.init_v, self.rem_v[:, :, st:st + take]), dim=-2)
            st += take
            live -= take
            self.init_full = self.init_k.shape[-2] == self.n_init
        while live - self.block_size >= self.n_local:
            live -= self.block_size
            for u in range(self.B):
                uk = self.rem_k[u, :, st:st + self.block_size].clone()
                uv = self.rem_v[u, :, st:st + self.block_size].clone()
                sc = self.rem_score[u, :, st:st + self.block_size].clone()
                rep, idx = self._representative(u, uk, sc)
                self.unit_trace.append(dict(unit=len(self.units[u]), row=u, score=sc, repr_idx=idx))
                self.units[u].append((uk, uv))
                self.reps[u].append(rep)
            self.n_units += 1
            st += self.block_size
        return st, ed

    # ------------------------------------------------------------------ append
    def append(self, q, k, v):
        if self.perhead:                                    # context_manager.py:690-704
            b0, h0, L = q.shape[0], q.shape[1], q.shape[2]
            rep = lambda t: t.repeat_interleave(h0 // t.shape[1], dim=1).reshape(b0 * h0, 1, L, -1)
            q, k, v = q.reshape(b0 * h0, 1, L, -1), rep(k), rep(v)
        if not self.ready:
            self._setup(q, k)
        L = q.shape[-2]
        self.win_k = torch.cat((self.win_k, k), dim=-2)
        self.win_v = torch.cat((self.win_v, v), dim=-2)
        kv_len = self.win_k.shape[-2]
        cur_st, cur_ed = 0, self.rem_k.shape[-2]
        self.rem_k = torch.cat((self.rem_k, k), dim=-2)
        self.rem_v = torch.cat((self.rem_v, v), dim=-2)
        self.rem_score = torch.cat((self.rem_score, torch.zeros(self.B, self.H, L, dtype=k.dtype)), dim=-1)
        gq = self.rope.one_angle(q, self.n_local)

        # context_manager.py:749-770: chunk boundaries at multiples of chunk_topk_calc, plus the tail
        use_chunks = self.chunk_topk_calc is not None and L > 1
        self._chunk_plan = None
        if use_chunks:
            per_chunk = self.chunk_topk_calc // self.exc_block_size
            cuts = [i * self.exc_block_size for i in range(0, L // self.exc_block_size + 1, per_chunk)]
            if cuts[-1] < L:
                cuts.append(L)
            cut_i = -1

        outs = []
        for st in range(0, L, self.exc_block_size):
            ed = min(st + self.exc_block_size, L)
            if use_chunks and cuts[cut_i + 1] < ed:
                cut_i += 1
                self._chunk_plan = self._retrieve_chunk(gq[:, :, cuts[cut_i]:cuts[cut_i + 1]])
                self._chunk_pos = 0
            kv_st = max(kv_len + st - L - self.n_local, 0)
            kv_ed = kv_len + ed - L
            o, ls = self._block(q[:, :, st:ed], self.win_k[:, :, kv_st:kv_ed],
                                self.win_v[:, :, kv_st:kv_ed], gq[:, :, st:ed], cur_st, cur_ed)
            outs.append(o)
            cur_st, cur_ed = self._after_block(ed - st, kv_ed - kv_st, ls, cur_st, cur_ed)
            if use_chunks:
                self._chunk_pos += 1

        self.length += L
        if self.win_k.shape[-2] >= self.n_local:
            self.win_k = self.win_k[:, :, -self.n_local:]
            self.win_v = self.win_v[:, :, -self.n_local:]
        assert cur_ed == self.rem_k.shape[-2]
        self.rem_k = self.rem_k[:, :, cur_st:]
        self.rem_v = self.rem_v[:, :, cur_st:]
        self.rem_score = self.rem_score[:, :, cur_st:]
        ret = torch.cat(outs, dim=-2)
        if self.perhead:
            ret = ret.reshape(b0, h0, L, -1)
        return ret
