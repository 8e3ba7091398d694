"""ContextManager: the streaming memory behind the "inf-llm" attention type.

Same constructor, ``append`` and ``size``/``length`` as
inf_llm/attention/context_manager.py:196-816, re-designed around absolute
stream positions and device-resident rings instead of torch.cat/trim:

* new tokens are written once into per-layer rings (raw K, RoPE'd K, V, fp32
  score track) by the prologue kernel, row = position % ring_cap; the local
  window and the "remainder" of the reference are index ranges of that ring;
* the local stage is one launch of the MFMA kernel over the ring with the
  causal sliding-window mask; the global stage is one launch over a page table
  of 64-key tiles (cached memory units, init tokens, overflow remainder) - the
  reference's global_buffer copies do not exist;
* both stages leave partials that the merge kernel joins into the joint
  softmax; the local score (probability column sums) is a third kernel that
  needs the merged log-sum-exp;
* memory units live in pinned host memory (always) and in a slab of
  ``max_cached_block`` device slots managed by the reference's lru / lru-s
  policy (plus fifo); misses are fetched with hipMemcpyAsync on a side stream.

State machine in absolute positions (context_manager.py:614-679 restated):
``cursor`` is the first token not yet carved, tokens [0, init_len) are the
attention sinks, unit u is tokens [n_init + u*bs, n_init + (u+1)*bs).
"""
import ctypes

import torch

from .. import ops
from ..ops import HEAD_DIM, KEY_TILE

_SIDE_STREAM = None          # one process-wide side stream, like GLOBAL_STREAM (context_manager.py:193)
_HOST_CHUNK_UNITS = 64       # units per pinned host allocation
_MAX_SPLITS = 16             # key splits of one attention stage
_NUM_CUS = 256               # MI355X


class CachePolicy:
    """Residency policy of one batch row (context_manager.py:246-265, 495-515).

    ``cached`` is an insertion-ordered dict unit -> value; eviction walks it in
    ascending value (stable), skipping the units selected for this block.
    """

    def __init__(self, capacity, strategy, score_decay):
        self.capacity, self.strategy, self.score_decay = capacity, strategy, score_decay
        self.cached = {}
        self.clock = 0
        self.slot_of = {}
        self.free = list(range(capacity - 1, -1, -1))

    def touch(self, selected):
        """Returns (misses, evicted) and updates values; slots of evicted units are freed."""
        misses = [b for b in selected if b not in self.cached]
        surplus = len(self.cached) - self.capacity + len(misses)
        evicted = []
        if surplus > 0:
            chosen = set(selected)
            for unit, _ in sorted(self.cached.items(), key=lambda kv: kv[1]):
                if unit not in chosen:
                    evicted.append(unit)
                if len(evicted) >= surplus:
                    break
            for unit in evicted:
                del self.cached[unit]
                self.free.append(self.slot_of.pop(unit))
        if self.strategy == "lru":
            self.clock += 1
            for b in selected:
                self.cached[b] = self.clock
        elif self.strategy == "fifo":
            self.clock += 1
            for b in selected:
                self.cached.setdefault(b, self.clock)
        else:                                   # lru-s
            for b in selected:
                self.cached[b] = 0
        assert len(self.cached) <= self.capacity, "topk exceeds max_cached_block"
        for b in misses:
            self.slot_of[b] = self.free.pop()
        return misses, evicted

    def add_scores(self, units, unit_scores):
        for u in self.cached:
            self.cached[u] = self.cached[u] * self.score_decay
        for u, s in zip(units, unit_scores):
            self.cached[u] += s


class ContextManager:
    def __init__(self, position_embedding, n_init, n_local, block_size, max_cached_block, topk, exc_block_size,
                 score_decay=None, fattn=False, repr_topk=1, cache_strategy="lru", chunk_topk_calc=None,
                 async_global_stream=False, pin_memory=False, faiss=False, perhead=False):
        assert exc_block_size <= n_local                       # no global token inside the input block
        assert cache_strategy in ("lru", "lru-s", "fifo")
        if faiss:
            raise NotImplementedError("the faiss representative store is not available in this build")
        if cache_strategy == "lru-s" and score_decay is None:
            raise ValueError("cache_strategy='lru-s' needs score_decay")
        self.length = 0
        self.position_embedding = position_embedding
        self.n_init, self.n_local = n_init, n_local
        self.block_size, self.max_cached_block = block_size, max_cached_block
        self.topk, self.exc_block_size = topk, exc_block_size
        self.score_decay, self.fattn, self.repr_topk = score_decay, fattn, repr_topk
        self.cache_strategy = cache_strategy
        self.chunk_topk_calc = chunk_topk_calc
        self.async_global_stream = async_global_stream
        self.pin_memory = pin_memory           # host copies are always pinned here
        self.perhead = perhead
        self.initialized = False
        self.load_count = 0
        self.record_trace = False
        self.kernel_timers = None          # dict(local=[], glob=[]) -> (start, end, n_queries, steady) event pairs
        self.trace_blocks, self.trace_units = [], []
        self.stats = dict(blocks=0, hits=0, misses=0, evictions=0)
        global _SIDE_STREAM
        if async_global_stream and _SIDE_STREAM is None and torch.cuda.is_available():
            _SIDE_STREAM = torch.cuda.Stream()

    # ------------------------------------------------------------------ setup
    def _init(self, q, k):
        B, H, _, D = q.shape
        Hkv = k.shape[1]
        dev = q.device
        if D != HEAD_DIM:
            raise ValueError(f"the HIP kernels are built for head_dim {HEAD_DIM}, got {D}")
        if self.topk > self.max_cached_block:
            raise ValueError("topk must not exceed max_cached_block")
        self.batch_size = self.num_units = B
        self.num_heads = self.unit_size = H
        self.num_heads_kv = self.unit_size_kv = Hkv
        self.dim_head = D
        self.dtype = q.dtype
        self.device = dev
        bs, exc = self.block_size, self.exc_block_size
        cap = self.n_local + exc + bs
        self.ring_cap = cap = (cap + KEY_TILE - 1) // KEY_TILE * KEY_TILE + KEY_TILE
        bf = dict(dtype=torch.bfloat16, device=dev)
        self.ring_k_raw = torch.zeros((B, Hkv, cap, D), **bf)
        self.ring_k_rot = torch.zeros((B, Hkv, cap, D), **bf)
        self.ring_v = torch.zeros((B, Hkv, cap, D), **bf)
        self.ring_score = torch.zeros((B, H, cap), dtype=torch.float32, device=dev)
        self.init_kv = torch.zeros((B, 2, Hkv, max(self.n_init, 1), D), **bf)
        self.slab = torch.zeros((B, self.max_cached_block, 2, Hkv, bs, D), **bf)
        self.reps = torch.zeros((B, 16, H * D), **bf)
        self.host_chunks = []
        self.policy = [CachePolicy(self.max_cached_block, self.cache_strategy, self.score_decay) for _ in range(B)]
        self.cursor = 0
        self.init_len = 0
        self.num_global_block = 0
        # workspaces of one execution block
        self.q_loc = torch.empty((B * H * exc * D,), **bf)
        self.q_glb = torch.empty((B * H * exc * D,), **bf)
        self.qbar = torch.empty((B, 1, H * D), dtype=torch.float32, device=dev)
        self.n_part = 2 * _MAX_SPLITS
        self.o_part = torch.empty((self.n_part * B * H * exc * D,), dtype=torch.float32, device=dev)
        self.lse_part = torch.empty((self.n_part * B * H * exc,), dtype=torch.float32, device=dev)
        self.lse = torch.empty((B * H * exc,), dtype=torch.float32, device=dev)
        self.topk_idx = torch.empty((B, max(self.topk, 1)), dtype=torch.int32, device=dev)
        self.topk_idx_host = torch.empty((B, max(self.topk, 1)), dtype=torch.int32, pin_memory=True)
        self.unit_scores = torch.empty((B, 16), dtype=torch.float32, device=dev)
        tiles_per_unit = (bs + KEY_TILE - 1) // KEY_TILE
        self.max_pages = (self.topk * tiles_per_unit + (self.n_init + KEY_TILE - 1) // KEY_TILE
                          + (exc + bs) // KEY_TILE + 3)
        self.page_bytes = ctypes.sizeof(ops.Page)
        self.pages_dev = torch.empty((B * self.max_pages * self.page_bytes,), dtype=torch.uint8, device=dev)
        self._page_stage = [torch.empty((B * self.max_pages * self.page_bytes,), dtype=torch.uint8, pin_memory=True)
                            for _ in range(4)]
        self._page_stage_evt = [None] * 4
        self._page_stage_cur = 0
        self._carve_stage = [None] * 4
        self._carve_evt = [None] * 4
        self._carve_cur = 0
        self.inv_freq = self.position_embedding.inv_freq.to(device=dev, dtype=torch.float32).contiguous()
        self.distance_scale = float(self.position_embedding.distance_scale)
        self._idx_event = torch.cuda.Event()
        self._global_done = None
        self.initialized = True

    def _splits(self, n_queries, n_tiles):
        """Key splits of one stage: enough workgroups to put about two on every CU, at least 8 tiles each."""
        G = self.unit_size // self.unit_size_kv
        wgs = ((n_queries + 31) // 32 * G + 3) // 4 * self.unit_size_kv * self.num_units
        want = (2 * _NUM_CUS + wgs - 1) // wgs
        return max(1, min(want, _MAX_SPLITS, n_tiles // 8))

    def size(self, *args, **kwargs):
        return self.length

    # ------------------------------------------------------------ host memory
    def _host_unit(self, unit):
        """Pinned host tensor [B, 2, Hkv, bs, D] of a unit."""
        chunk, idx = divmod(unit, _HOST_CHUNK_UNITS)
        while chunk >= len(self.host_chunks):
            self.host_chunks.append(torch.empty(
                (_HOST_CHUNK_UNITS, self.num_units, 2, self.unit_size_kv, self.block_size, self.dim_head),
                dtype=torch.bfloat16, pin_memory=True))
        return self.host_chunks[chunk][idx]

    def _copy_stream(self):
        return _SIDE_STREAM if self.async_global_stream else torch.cuda.current_stream()

    # -------------------------------------------------------------- retrieval
    def _retrieve(self):
        """Unit ids per batch row for the current block (context_manager.py:366-383)."""
        N, B = self.num_global_block, self.num_units
        if N <= self.topk:
            return [list(range(N)) for _ in range(B)]
        if self.unit_scores.shape[1] < N:
            self.unit_scores = torch.empty((B, self.reps.shape[1]), dtype=torch.float32, device=self.device)
        for u in range(B):
            ops.score_topk(self.reps[u], N, self.qbar[u], self.topk, self.unit_scores[u], self.topk_idx[u])
        self.topk_idx_host.copy_(self.topk_idx, non_blocking=True)
        self._idx_event.record()
        self._idx_event.synchronize()          # the one host sync of a block (context_manager.py:163)
        return self.topk_idx_host.tolist()

    # ------------------------------------------------------------- page table
    def _build_pages(self, selected, b1):
        B, bs, D = self.num_units, self.block_size, self.dim_head
        esz = 2
        unit_stride = self.unit_size_kv * bs * D                       # K -> V inside a slot
        overflow_end = max(b1 - self.n_local, self.cursor)
        rows = []
        for u in range(B):
            ent = []
            slab_u = self.slab[u]
            for unit in selected[u]:
                slot = self.policy[u].slot_of[unit]
                k_addr = slab_u[slot].data_ptr()
                for t0 in range(0, bs, KEY_TILE):
                    ent.append((k_addr + t0 * D * esz, k_addr + (unit_stride + t0 * D) * esz, bs * D, min(KEY_TILE, bs - t0)))
            ik = self.init_kv[u, 0].data_ptr()
            iv = self.init_kv[u, 1].data_ptr()
            ilen = self.init_kv.shape[3]
            for t0 in range(0, self.init_len, KEY_TILE):
                ent.append((ik + t0 * D * esz, iv + t0 * D * esz, ilen * D, min(KEY_TILE, self.init_len - t0)))
            rk, rv = self.ring_k_raw[u].data_ptr(), self.ring_v[u].data_ptr()
            pos = self.cursor
            while pos < overflow_end:
                row = pos % self.ring_cap
                n = min(KEY_TILE, overflow_end - pos, self.ring_cap - row)
                ent.append((rk + row * D * esz, rv + row * D * esz, self.ring_cap * D, n))
                pos += n
            rows.append(ent)
        n_pages = len(rows[0])
        assert all(len(r) == n_pages for r in rows) and n_pages <= self.max_pages
        if n_pages == 0:
            return 0
        arr = ops.make_pages([e for r in rows for e in r])
        slot = self._page_stage_cur
        self._page_stage_cur = (slot + 1) % len(self._page_stage)
        if self._page_stage_evt[slot] is not None:
            self._page_stage_evt[slot].synchronize()
        nbytes = B * n_pages * self.page_bytes
        ctypes.memmove(self._page_stage[slot].data_ptr(), arr, nbytes)
        ops.copy_async(self.pages_dev, self._page_stage[slot], nbytes, 1)
        evt = self._page_stage_evt[slot] or torch.cuda.Event()
        evt.record()
        self._page_stage_evt[slot] = evt
        return n_pages

    # -------------------------------------------------------- one exec block
    def _block(self, q, k, v, out, b0):
        B, H, Hkv, D = self.num_units, self.unit_size, self.unit_size_kv, self.dim_head
        n = q.shape[2]
        b1 = b0 + n
        main = torch.cuda.current_stream()
        q_loc = self.q_loc[:B * H * n * D].view(B, H, n, D)
        q_glb = self.q_glb[:B * H * n * D].view(B, H, n, D)
        o_part = self.o_part[:self.n_part * B * H * n * D].view(self.n_part, B, H, n, D)
        lse_part = self.lse_part[:self.n_part * B * H * n].view(self.n_part, B, H, n)
        lse = self.lse[:B * H * n].view(B, H, n)

        ops.ingest(q, k, v, b0, self.n_local - 1, self.inv_freq, self.distance_scale,
                   self.ring_k_raw, self.ring_k_rot, self.ring_v, self.ring_score, q_loc, q_glb)
        ops.block_mean(q_glb, B, H, n, n, self.qbar)
        # local stage first: it keeps the GPU busy while the host resolves the retrieval
        lo = max(b0 - self.n_local, 0)
        tm = self.kernel_timers
        if tm is not None:
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
        sl = self._splits(n, (b1 - lo + KEY_TILE - 1) // KEY_TILE)
        ops.attn_stage_linear(q_loc, self.ring_k_rot, self.ring_v, o_part[0:sl], lse_part[0:sl], cap=self.ring_cap,
                              j_lo=lo, j_hi=b1, mask=ops.MASK_WINDOW, offset=b0, window=self.n_local, nsplit=sl)
        if tm is not None:
            e1.record()
            tm["local"].append((e0, e1, n, n == self.exc_block_size and lo == b0 - self.n_local))

        selected = self._retrieve()
        copy_stream = self._copy_stream()
        fetched = False
        for u in range(B):
            misses, evicted = self.policy[u].touch(selected[u])
            self.stats["hits"] += len(selected[u]) - len(misses)
            self.stats["misses"] += len(misses)
            self.stats["evictions"] += len(evicted)
            for unit in misses:
                if not fetched and copy_stream is not main and self._global_done is not None:
                    copy_stream.wait_event(self._global_done)   # the slot may still be read by the previous block
                fetched = True
                slot = self.policy[u].slot_of[unit]
                src = self._host_unit(unit)[u]
                ops.copy_async(self.slab[u, slot], src, src.numel() * 2, 1, copy_stream.cuda_stream)
        if fetched and copy_stream is not main:
            main.wait_stream(copy_stream)
        if self.cache_strategy == "lru":
            self.load_count += 1

        n_pages = self._build_pages(selected, b1)
        if n_pages > 0:
            if tm is not None:
                e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                e0.record()
            sg = self._splits(n, n_pages)
            ops.attn_stage_paged(q_glb, self.pages_dev, n_pages, Hkv, o_part[sl:sl + sg], lse_part[sl:sl + sg], nsplit=sg)
            if tm is not None:
                e1.record()
                tm["glob"].append((e0, e1, n, n == self.exc_block_size and self.num_global_block >= self.topk))
            if copy_stream is not main:
                if self._global_done is None:
                    self._global_done = torch.cuda.Event()
                self._global_done.record(main)
            ops.attn_merge(o_part, lse_part, sl + sg, out, lse)
        else:
            ops.attn_merge(o_part, lse_part, sl, out, lse)
        ops.local_score(q_loc, self.ring_k_rot, lse, self.ring_score, cap=self.ring_cap, j_lo=lo, j_hi=b1,
                        mask=ops.MASK_WINDOW, offset=b0, window=self.n_local, accumulate=True, score_cap=self.ring_cap)
        if self.cache_strategy == "lru-s":
            raise NotImplementedError("lru-s needs the per-unit global score kernel")
        if self.record_trace:
            self.trace_blocks.append(dict(b0=b0, b1=b1, selected=[sorted(s) for s in selected], n_units=self.num_global_block,
                                          init_len=self.init_len, n_pages=n_pages))
        self.stats["blocks"] += 1
        self._after_block(b1)

    def _after_block(self, b1):
        """Init peeling and unit carving (context_manager.py:614-679) in absolute positions."""
        B, H, Hkv, D, bs = self.num_units, self.unit_size, self.unit_size_kv, self.dim_head, self.block_size
        live = b1 - self.cursor
        if self.init_len < self.n_init and live > self.n_local:
            take = min(self.n_init - self.init_len, live - self.n_local)
            ilen = self.init_kv.shape[3]
            for which, ring in ((0, self.ring_k_raw), (1, self.ring_v)):
                ops.gather_rows(ring, self.cursor, take, self.init_kv[:, which, :, self.init_len].data_ptr(),
                                2 * Hkv * ilen * D, ilen * D)
            self.init_len += take
            self.cursor += take
            live -= take
        c = max((live - self.n_local) // bs, 0)
        if c == 0:
            return
        N = self.num_global_block
        if N + c > self.reps.shape[1]:
            grown = torch.zeros((B, max(2 * self.reps.shape[1], N + c), H * D), dtype=torch.bfloat16, device=self.device)
            grown[:, :N] = self.reps[:, :N]
            self.reps = grown
        idx_out = torch.empty((B, c, H, self.repr_topk), dtype=torch.int32, device=self.device) if self.record_trace else None
        ops.repr_keys(self.ring_score, self.ring_k_raw, self.cursor, bs, c, self.repr_topk,
                      self.reps[:, N], self.reps.stride(0), self.reps.stride(1), idx_out)
        if self.record_trace:
            self.trace_units.append((N, c, idx_out))
        # carve: ring -> contiguous device staging -> pinned host (the units' permanent home)
        slot = self._carve_cur
        self._carve_cur = (slot + 1) % len(self._carve_stage)
        if self._carve_evt[slot] is not None:
            self._carve_evt[slot].synchronize()
        stage = self._carve_stage[slot]
        if stage is None or stage.shape[0] < c:
            stage = torch.empty((max(c, 4), B, 2, Hkv, bs, D), dtype=torch.bfloat16, device=self.device)
            self._carve_stage[slot] = stage
        for which, ring in ((0, self.ring_k_raw), (1, self.ring_v)):
            ops.gather_rows(ring, self.cursor, c * bs, stage[0, 0, which].data_ptr(), stage.stride(1), stage.stride(3),
                            unit_rows=bs, out_su=stage.stride(0))
        main = torch.cuda.current_stream()
        copy_stream = self._copy_stream()
        if copy_stream is not main:
            copy_stream.wait_stream(main)
        unit_bytes = B * 2 * Hkv * bs * D * 2
        for i in range(c):
            ops.copy_async(self._host_unit(N + i), stage[i], unit_bytes, 2, copy_stream.cuda_stream)
        evt = self._carve_evt[slot] or torch.cuda.Event()
        evt.record(copy_stream)
        self._carve_evt[slot] = evt
        self.cursor += c * bs
        self.num_global_block += c

    # ----------------------------------------------------------------- append
    def append(self, local_q, local_k, local_v, global_q, global_k, global_v):
        if not (global_q is local_q and global_k is local_k and global_v is local_v):
            if not (global_q.data_ptr() == local_q.data_ptr() and global_k.data_ptr() == local_k.data_ptr()
                    and global_v.data_ptr() == local_v.data_ptr()):
                raise ValueError("local and global q/k/v must be the same tensors (as inf_llm_forward passes them)")
        q, k, v = local_q, local_k, local_v
        if q.dtype != torch.bfloat16:
            raise TypeError(f"the HIP path computes in bfloat16; got {q.dtype}")
        assert q.dim() == 4 and q.is_cuda
        batch_size, input_length = q.size(0), q.size(-2)
        for t in (q, k, v):
            assert t.size(0) == batch_size and t.size(2) == input_length and t.size(3) == q.size(3)
        if self.perhead:                                        # context_manager.py:690-704
            heads, heads_kv = q.size(1), k.size(1)
            rep = lambda t: (t.reshape(batch_size, heads_kv, 1, input_length, -1)
                              .expand(batch_size, heads_kv, heads // heads_kv, input_length, -1)
                              .reshape(batch_size * heads, 1, input_length, -1))
            q, k, v = q.reshape(batch_size * heads, 1, input_length, -1), rep(k), rep(v)
        if not self.initialized:
            self._init(q, k)
        assert q.shape[:2] == (self.num_units, self.unit_size) and k.shape[1] == self.unit_size_kv
        q, k, v = ops._bf16_4d(q, "q"), ops._bf16_4d(k, "k"), ops._bf16_4d(v, "v")
        out = torch.empty((self.num_units, self.unit_size, input_length, self.dim_head), dtype=torch.bfloat16, device=q.device)
        if self.chunk_topk_calc is not None and input_length > 1:
            raise NotImplementedError("chunk_topk_calc is not implemented yet")
        for st in range(0, input_length, self.exc_block_size):
            ed = min(st + self.exc_block_size, input_length)
            self._block(q[:, :, st:ed], k[:, :, st:ed], v[:, :, st:ed], out[:, :, st:ed], self.length + st)
        self.length += input_length
        if self.perhead:
            out = out.view(batch_size, heads, input_length, -1)
        return out

    # ----------------------------------------------------------------- tracing
    def trace_repr_indices(self):
        """{unit: int tensor [B, H, repr_topk]} of the keys chosen as representatives (needs record_trace)."""
        res = {}
        for first, count, idx in self.trace_units:
            host = idx.cpu()
            for i in range(count):
                res[first + i] = host[:, i]
        return res
