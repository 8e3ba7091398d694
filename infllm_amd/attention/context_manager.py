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
  policy (plus fifo; native, infllm_cache_*); the misses of a block are moved
  by the DMA engines (short blocks: read from the pinned pages by one kernel
  on a side stream), for lru / fifo starting from the selection's candidates a
  block ahead of the selection itself (``fetch_ahead``).

This module keeps the state machine, in absolute positions
(context_manager.py:614-679 restated): ``cursor`` is the first token not yet
carved, tokens [0, init_len) are the attention sinks, unit u is tokens
[n_init + u*bs, n_init + (u+1)*bs).  The device work of one execution block is
issued by three native calls: infllm_block_front, infllm_block_select (the one
host wait, for the retrieved unit ids, which overlaps the local stage; then
cache policy and fetch) and infllm_block_back, plus infllm_block_prefetch for
the next block.
"""
import ctypes
import os

import torch

from .. import _lib
from .._lib import BackArgs, FrontArgs, LayerDesc, check
from ..ops import HEAD_DIM, KEY_TILE

from ._rows import check_head_dim, narrow as _narrow, wide_inv_freq, widen as _widen

_SIDE_STREAM = None          # one process-wide side stream, like GLOBAL_STREAM (context_manager.py:193)
_CALL_BUFFERS = {}           # (device, stream, geometry) -> the buffers of a call prepared in one go, see _bind_call_buffers
_HOST_CHUNK_UNITS = 64       # units per pinned host allocation
_MAX_SPLITS = 16             # key splits of one attention stage
_NUM_CUS = 256               # MI355X
_PAGE_SLOTS = 4
_CARVE_SLOTS = 4             # staging slots of the carve, used in turn (more of them serve more misses on the device - 16: 18 %,
                             # 64: 57 % of the benchmark stream's - but the stream is no faster for it, measured)


class CachePolicy:
    """Residency policy of one batch row (context_manager.py:246-265, 495-515): a handle on the native
    object (infllm_cache_*), which ContextManager also drives directly from infllm_block_select.

    ``cached`` is the reference's insertion-ordered dict unit -> value; eviction walks it in
    ascending value (stable), skipping the units selected for this block.
    """

    def __init__(self, capacity, strategy, score_decay):
        self.capacity, self.strategy, self.score_decay = capacity, strategy, score_decay
        self._lib = _lib.load()
        self.handle = self._lib.infllm_cache_create(capacity, _lib.CACHE_STRATEGY[strategy],
                                                    float(score_decay) if score_decay is not None else 0.0)
        if not self.handle:
            raise _lib.InfLLMHipError((self._lib.infllm_last_error() or b"").decode())
        self.evicted_log = None             # set to a list to record the evictions of every block
        self._units = (ctypes.c_int32 * capacity)()
        self._slots = (ctypes.c_int32 * capacity)()
        self._values = (ctypes.c_double * capacity)()

    def __del__(self):
        if getattr(self, "handle", None):
            self._lib.infllm_cache_destroy(self.handle)
            self.handle = None

    def touch(self, selected):
        """Returns (misses, evicted) and updates values; slots of evicted units are freed."""
        n = len(selected)
        assert n <= self.capacity, "topk exceeds max_cached_block"
        sel = (ctypes.c_int32 * max(n, 1))(*selected)
        slots, mu, ms = ((ctypes.c_int32 * max(n, 1))() for _ in range(3))
        ev, n_ev = (ctypes.c_int32 * self.capacity)(), ctypes.c_int32(0)
        n_miss = self._lib.infllm_cache_touch(self.handle, sel, n, slots, mu, ms, ev, ctypes.byref(n_ev))
        if n_miss < 0:
            check(n_miss, "infllm_cache_touch")
        evicted = list(ev[:n_ev.value])
        if self.evicted_log is not None:
            self.evicted_log.append(evicted)
        return list(mu[:n_miss]), evicted

    def add_scores(self, units, unit_scores):
        n = len(units)
        check(self._lib.infllm_cache_add_scores(self.handle, (ctypes.c_int32 * max(n, 1))(*units),
                                                (ctypes.c_double * max(n, 1))(*unit_scores[:n]), n), "infllm_cache_add_scores")

    def _residents(self):
        n = self._lib.infllm_cache_residents(self.handle, self._units, self._values, self._slots, self.capacity)
        if n < 0:
            check(n, "infllm_cache_residents")
        return n

    @property
    def cached(self):
        n = self._residents()
        as_int = self.strategy != "lru-s"
        return {self._units[i]: (int(self._values[i]) if as_int else self._values[i]) for i in range(n)}

    @property
    def slot_of(self):
        n = self._residents()
        return {self._units[i]: self._slots[i] for i in range(n)}

    @property
    def free(self):
        used = set(self.slot_of.values())
        return [s for s in range(self.capacity) if s not in used]


class ContextManager:
    select_in_steps = False     # True: drive wait / policy / fetch from here (slower), instead of infllm_block_select
    fetch_ahead = True          # start the next block's fetch from its candidates (infllm_block_prefetch)
    call_tokens = 8192          # tokens of an append() call prepared in one go (prologue, mean queries and the local
                                # stage of all their blocks: infllm_call_front); 0: every block runs its own.
                                # INFLLM_CALL_TOKENS overrides it.  Needs exc_block_size to be a multiple of 32.
    local_group_blocks = 2      # blocks of a prepared call per launch of the local stage (INFLLM_LOCAL_GROUP overrides it)

    def __init__(self, position_embedding, n_init, n_local, block_size, max_cached_block, topk, exc_block_size,
                 score_decay=None, fattn=False, repr_topk=1, cache_strategy="lru", chunk_topk_calc=None,
                 async_global_stream=False, pin_memory=False, faiss=False, perhead=False):
        assert exc_block_size <= n_local                       # no global token inside the input block
        assert cache_strategy in ("lru", "lru-s", "fifo")
        if faiss:
            raise NotImplementedError("the faiss representative store is not available in this build")
        if cache_strategy == "lru-s":
            assert score_decay is not None, "cache_strategy='lru-s' needs score_decay"
        if chunk_topk_calc is not None:
            assert chunk_topk_calc >= exc_block_size, "chunk_topk_calc must cover at least one execution block"
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
        self.trace_blocks, self.trace_units = [], []
        self._call_scores = None      # [blocks of a call, B, units]: scores of every unit under every block's mean query
        self._host_copies_open = False
        self.stats = dict(blocks=0, hits=0, misses=0, evictions=0)
        self._layer = None
        self._timing_cap, self._timing_stride = 0, 1
        self._mass_units = None                # lru-s: selections of the block whose unit masses are still on the device
        global _SIDE_STREAM
        if async_global_stream and _SIDE_STREAM is None and torch.cuda.is_available():
            _SIDE_STREAM = torch.cuda.Stream()

    def __del__(self):
        layer, self._layer = getattr(self, "_layer", None), None
        if layer:
            try:
                _lib.load().infllm_layer_destroy(layer)       # waits for this layer's own work, not for the device
            except Exception:
                pass

    # ------------------------------------------------------------------ setup
    def _init(self, q, k):
        B, H, _, D = q.shape
        Hkv = k.shape[1]
        dev = q.device
        assert D == HEAD_DIM                                    # rows arrive widened (see _widen)
        if self.topk > self.max_cached_block:
            raise ValueError("topk must not exceed max_cached_block")
        if self.topk > 64:
            raise ValueError("this build selects at most 64 units per block (topk <= 64)")
        if self.repr_topk > self.block_size:
            raise ValueError("repr_topk must not exceed block_size")
        self.batch_size = self.num_units = B
        self.num_heads = self.unit_size = H
        self.num_heads_kv = self.unit_size_kv = Hkv
        self.head_width = D                                     # of the rows the kernels see; self.dim_head is the caller's
        self.dtype = q.dtype
        self.device = dev
        bs, exc, topk = self.block_size, self.exc_block_size, self.topk
        ct = int(os.environ.get("INFLLM_CALL_TOKENS", self.call_tokens))
        self._call_tokens = min(ct, 16 * exc) // exc * exc if (ct >= exc and exc % 32 == 0) else 0
        # the rings hold the local window, the remainder that waits to fill a unit, and what is prepared ahead of the
        # block being attended: one block, or the rest of a call prepared in one go
        cap = self.n_local + exc + bs + max(exc, self._call_tokens)
        self.ring_cap = cap = (cap + KEY_TILE - 1) // KEY_TILE * KEY_TILE + KEY_TILE
        bf = dict(dtype=torch.bfloat16, device=dev)
        f32 = dict(dtype=torch.float32, device=dev)
        self.ring_k_raw = torch.zeros((B, Hkv, cap, D), **bf)
        self.ring_k_rot = torch.zeros((B, Hkv, cap, D), **bf)
        self.ring_v = torch.zeros((B, Hkv, cap, D), **bf)
        self.ring_score = torch.zeros((B, H, cap), **f32)
        self.init_kv = torch.zeros((B, 2, Hkv, max(self.n_init, 1), D), **bf)
        self.slab = torch.zeros((B, self.max_cached_block, 2, Hkv, bs, D), **bf)
        self.reps = torch.zeros((B, 16, H * D), **bf)
        self.unit_scores = torch.empty((B, 16), **f32)
        self.host_chunks, self._host_base, self._host_dev_base = [], [], []
        self._chunk_base = (ctypes.c_uint64 * 64)()           # device-visible chunk addresses, as the native side reads them
        self.policy = [CachePolicy(self.max_cached_block, self.cache_strategy, self.score_decay) for _ in range(B)]
        if self.record_trace:
            for pol in self.policy:
                pol.evicted_log = []
        self.cursor = 0
        self.init_len = 0
        self.num_global_block = 0
        # workspaces of one execution block
        self.q_loc = torch.empty((2, B * H * exc * D), **bf)        # two slots: this block / the one prepared ahead
        self.q_glb = torch.empty((2, B * H * exc * D), **bf)
        self.qbar = torch.empty((2, B, H * D), **f32)
        self.qpart = torch.empty((2, B, (exc + 15) // 16, H * D), **f32)
        n_part = 2 * _MAX_SPLITS
        self.o_part = torch.empty((n_part * B * H * exc * D,), dtype=torch.float16, device=self.device)
        self.lse_part = torch.empty((n_part * B * H * exc,), **f32)
        self.lse = torch.empty((B * H * exc,), **f32)
        self.topk_idx = torch.zeros((B, max(topk, 1)), dtype=torch.int32, device=dev)
        self.topk_idx_host = torch.zeros((B, max(topk, 1)), dtype=torch.int32, pin_memory=True)
        tiles_per_unit = (bs + KEY_TILE - 1) // KEY_TILE
        self.max_pages = topk * tiles_per_unit + (self.n_init + KEY_TILE - 1) // KEY_TILE + (exc + bs) // KEY_TILE + 3
        page_bytes = ctypes.sizeof(_lib.Page)
        self.pages_dev = torch.empty((B * self.max_pages * page_bytes,), dtype=torch.uint8, device=dev)
        self.pages_host = torch.empty((_PAGE_SLOTS * B * self.max_pages * page_bytes,), dtype=torch.uint8, pin_memory=True)
        self.max_carve = (exc + self.n_init) // bs + 2
        self.carve_stage = torch.empty((_CARVE_SLOTS, self.max_carve, B, 2, Hkv, bs, D), **bf)
        if self.position_embedding.inv_freq.numel() != self.dim_head // 2:
            raise ValueError(f"the rotary embedding is built for head_dim {2 * self.position_embedding.inv_freq.numel()}, "
                             f"the heads have {self.dim_head}")
        self.inv_freq = wide_inv_freq(self.position_embedding.inv_freq, dev)
        self.slot_bytes = 2 * Hkv * bs * D * 2              # one unit of one batch row
        self.unit_bytes = B * self.slot_bytes               # one unit, all batch rows

        d = LayerDesc()
        d.B, d.H, d.Hkv = B, H, Hkv
        d.n_local, d.n_init, d.block_size, d.exc = self.n_local, self.n_init, bs, exc
        d.topk, d.repr_topk, d.max_cached = topk, self.repr_topk, self.max_cached_block
        d.max_splits, d.num_cus, d.ring_cap = _MAX_SPLITS, _NUM_CUS, cap
        d.d_ring_k_raw, d.d_ring_k_rot = self.ring_k_raw.data_ptr(), self.ring_k_rot.data_ptr()
        d.d_ring_v, d.d_ring_score = self.ring_v.data_ptr(), self.ring_score.data_ptr()
        d.d_init_kv, d.init_cap, d.d_slab = self.init_kv.data_ptr(), self.init_kv.shape[3], self.slab.data_ptr()
        d.d_q_loc, d.d_q_glb, d.d_qbar = self.q_loc.data_ptr(), self.q_glb.data_ptr(), self.qbar.data_ptr()
        d.d_qpart = self.qpart.data_ptr()
        d.d_o_part, d.d_lse_part, d.d_lse = self.o_part.data_ptr(), self.lse_part.data_ptr(), self.lse.data_ptr()
        self._lib = _lib.load()
        # the top-k kernel writes the ids straight into pinned host memory (no copy in the chain)
        d.d_topk_idx = self._lib.infllm_host_device_pointer(self.topk_idx_host.data_ptr())
        d.h_topk_idx = None
        if not d.d_topk_idx:
            d.d_topk_idx, d.h_topk_idx = self.topk_idx.data_ptr(), self.topk_idx_host.data_ptr()
        else:                                      # the host polls a sequence number stored behind the ids
            self.topk_flag_host = torch.zeros((16,), dtype=torch.int32, pin_memory=True)
            d.d_topk_flag = self._lib.infllm_host_device_pointer(self.topk_flag_host.data_ptr())
            d.h_topk_flag = self.topk_flag_host.data_ptr() if d.d_topk_flag else None
        d.d_pages, d.h_pages = self.pages_dev.data_ptr(), self.pages_host.data_ptr()
        d.max_pages, d.page_slots = self.max_pages, _PAGE_SLOTS
        d.d_carve_stage, d.max_carve, d.carve_slots = self.carve_stage.data_ptr(), self.max_carve, _CARVE_SLOTS
        d.d_inv_freq = self.inv_freq.data_ptr()
        d.distance_scale = float(self.position_embedding.distance_scale)
        d.softmax_scale = 1.0 / (self.dim_head ** 0.5)
        self._lib = _lib.load()
        self._layer = self._lib.infllm_layer_create(ctypes.byref(d))
        if not self._layer:
            raise _lib.InfLLMHipError("infllm_layer_create failed: " + (self._lib.infllm_last_error() or b"").decode())
        if self._timing_cap:
            check(self._lib.infllm_layer_timing(self._layer, self._timing_cap, self._timing_stride), "infllm_layer_timing")
        self._call_stream = None               # stream the call buffers were taken for (they are bound at the first append)
        # argument blocks and host arrays reused by every block
        self._fa, self._ba = FrontArgs(), BackArgs()
        self._sel_slots = (ctypes.c_int32 * (B * max(topk, 1)))()
        self._miss_row = (ctypes.c_int32 * (B * max(topk, 1)))()
        self._miss_slot = (ctypes.c_int32 * (B * max(topk, 1)))()
        self._miss_unit = (ctypes.c_int32 * (B * max(topk, 1)))()
        self._miss_src = (ctypes.c_void_p * (B * max(topk, 1)))()
        self._carve_dst = (ctypes.c_void_p * self.max_carve)()
        ba = self._ba
        ba.h_sel_slots = ctypes.addressof(self._sel_slots)
        ba.h_miss_row, ba.h_miss_slot = ctypes.addressof(self._miss_row), ctypes.addressof(self._miss_slot)
        ba.h_miss_unit = ctypes.addressof(self._miss_unit)
        ba.h_miss_src, ba.h_carve_dst = ctypes.addressof(self._miss_src), ctypes.addressof(self._carve_dst)
        if self.cache_strategy == "lru-s":
            # context_manager.py:454-470: per-unit attention mass of every block, read back by the host
            self.mass_host = torch.zeros((B, max(topk, 1)), dtype=torch.float32, pin_memory=True)
            self.mass_scratch = torch.empty((B, max(topk, 1), H, bs), **f32)
            ba.d_unit_mass = self._lib.infllm_host_device_pointer(self.mass_host.data_ptr())
            if not ba.d_unit_mass:
                raise _lib.InfLLMHipError("pinned host memory is not device-mapped: " + (self._lib.infllm_last_error() or b"").decode())
            ba.d_mass_scratch = self.mass_scratch.data_ptr()
        # selection -> cache policy -> fetch runs natively (infllm_block_select) on these arrays
        n_ids = B * max(topk, 1)
        self._sel_ids = (ctypes.c_int32 * n_ids)()
        self._evicted = (ctypes.c_int32 * n_ids)()
        self._n_evicted, self._n_miss_row = (ctypes.c_int32 * B)(), (ctypes.c_int32 * B)()
        self._caches = (ctypes.c_void_p * B)(*[pol.handle for pol in self.policy])
        sa = self._sa = _lib.SelectArgs()
        sa.caches = ctypes.addressof(self._caches)
        sa.h_chunk_base, sa.n_chunks, sa.units_per_chunk = ctypes.addressof(self._chunk_base), 0, _HOST_CHUNK_UNITS
        sa.unit_bytes, sa.row_bytes = self.unit_bytes, self.slot_bytes
        sa.h_sel_slots = ba.h_sel_slots
        sa.h_miss_row, sa.h_miss_slot, sa.h_miss_unit, sa.h_miss_src = ba.h_miss_row, ba.h_miss_slot, ba.h_miss_unit, ba.h_miss_src
        sa.h_evicted, sa.h_n_evicted, sa.h_n_miss = (ctypes.addressof(self._evicted), ctypes.addressof(self._n_evicted),
                                                      ctypes.addressof(self._n_miss_row))
        self._sa_ref = ctypes.byref(sa)
        self._fa_ref, self._ba_ref = ctypes.byref(self._fa), ctypes.byref(self._ba)
        self.initialized = True

    def _bind_call_buffers(self, stream):
        """Buffers of a call prepared in one go: the rotated queries of up to call_tokens tokens, the blocks' mean
        queries and the local stage's partial rows.  They are dead between append() calls, so the layers that work on
        one stream (one after the other, as the layers of a model do) share one set."""
        B, H, D, exc, T = self.num_units, self.unit_size, self.head_width, self.exc_block_size, self._call_tokens
        group = int(os.environ.get("INFLLM_LOCAL_GROUP", self.local_group_blocks))
        blocks = max(8, 4 * group)            # partial rows: two groups of blocks, up to two key splits each
        dev = self.device.index if self.device.index is not None else torch.cuda.current_device()
        key = (dev, stream, B, H, D, T, exc, blocks)
        buf = _CALL_BUFFERS.get(key)
        if buf is None:
            bf = dict(dtype=torch.bfloat16, device=self.device)
            f32 = dict(dtype=torch.float32, device=self.device)
            buf = _CALL_BUFFERS[key] = dict(
                q_loc=torch.empty((B, H, T, D), **bf), q_glb=torch.empty((B, H, T, D), **bf),
                qpart=torch.empty((B, (T + 15) // 16, H * D), **f32), qbar=torch.empty((T // exc, B, H * D), **f32),
                o_part=torch.empty((blocks * B * H * exc, D), dtype=torch.float16, device=self.device),
                lse_part=torch.empty((blocks * B * H * exc,), **f32))
        self._call_buf = buf
        bd = _lib.BatchDesc()
        bd.d_q_loc, bd.d_q_glb = buf["q_loc"].data_ptr(), buf["q_glb"].data_ptr()
        bd.d_qpart, bd.d_qbar = buf["qpart"].data_ptr(), buf["qbar"].data_ptr()
        bd.d_o_part, bd.d_lse_part = buf["o_part"].data_ptr(), buf["lse_part"].data_ptr()
        bd.part_rows, bd.max_tokens, bd.group_blocks = blocks * B * H * exc, T, group
        check(self._lib.infllm_layer_set_batch(self._layer, ctypes.byref(bd)), "infllm_layer_set_batch")
        self._call_stream = stream

    def size(self, *args, **kwargs):
        return self.length

    # ------------------------------------------------------------ host memory
    def _host_unit_addr(self, unit):
        """Address of the pinned host copy [B, 2, Hkv, bs, D] of a unit."""
        chunk, idx = divmod(unit, _HOST_CHUNK_UNITS)
        while chunk >= len(self.host_chunks):
            t = torch.empty((_HOST_CHUNK_UNITS, self.num_units, 2, self.unit_size_kv, self.block_size, self.head_width),
                            dtype=torch.bfloat16, pin_memory=True)
            self.host_chunks.append(t)
            self._host_base.append(t.data_ptr())
            dev = self._lib.infllm_host_device_pointer(t.data_ptr())       # address the fetch kernel reads through
            if not dev:
                raise _lib.InfLLMHipError((self._lib.infllm_last_error() or b"").decode())
            self._host_dev_base.append(dev)
            if len(self._host_dev_base) > len(self._chunk_base):
                grown = (ctypes.c_uint64 * (2 * len(self._chunk_base)))()
                grown[:len(self._chunk_base)] = self._chunk_base[:]
                self._chunk_base = grown
                self._sa.h_chunk_base = ctypes.addressof(grown)
            self._chunk_base[len(self._host_dev_base) - 1] = dev
            self._sa.n_chunks = len(self._host_dev_base)
        return self._host_base[chunk] + idx * self.unit_bytes

    def _host_unit_rows(self, unit):
        chunk, idx = divmod(unit, _HOST_CHUNK_UNITS)
        return self.host_chunks[chunk][idx]

    def _finish_host_copies(self):
        """append() leaves the copy of the units it carved last to their pinned home in flight; this sees it through."""
        if self._host_copies_open and self._layer:
            check(self._lib.infllm_layer_flush(self._layer, self._copy_raw), "infllm_layer_flush")
            torch.cuda.synchronize(self.device)            # (the copy-stream form of that copy is only ordered by its stream)
            self._host_copies_open = False

    def host_unit(self, unit):
        """Pinned host tensor [B, 2, Hkv, bs, D] of a carved unit (K at index 0, V at 1); for heads narrower than 128 a
        copy with the real dimensions picked out."""
        self._finish_host_copies()
        return _narrow(self._host_unit_rows(unit), self.dim_head)

    def rep_rows(self, row, lo, hi):
        """Representatives of units [lo, hi) of batch row `row` as a CPU fp32 tensor [hi - lo, H * D]."""
        r = self.reps[row, lo:hi].view(hi - lo, self.unit_size, self.head_width)
        return _narrow(r, self.dim_head).reshape(hi - lo, -1).float().cpu()

    # ----------------------------------------------------------------- timing
    def enable_timing(self, capacity, stride=1):
        """Event-time every `stride`-th local / global stage launch (up to `capacity` of each) for benchmarks."""
        self._timing_cap, self._timing_stride = capacity, stride
        if self._layer:
            check(self._lib.infllm_layer_timing(self._layer, capacity, stride), "infllm_layer_timing")

    def prefetch_stats(self):
        """(guesses made, guesses that turned out to be the selection) of the fetch ahead of the selection."""
        issued, confirmed = ctypes.c_int64(0), ctypes.c_int64(0)
        if self._layer:
            check(self._lib.infllm_layer_prefetch_stats(self._layer, ctypes.byref(issued), ctypes.byref(confirmed)),
                  "infllm_layer_prefetch_stats")
        return issued.value, confirmed.value

    def staged_units(self):
        """Missed units that were copied from a carve staging slot instead of coming from pinned host memory."""
        return int(self._lib.infllm_layer_staged_units(self._layer)) if self._layer else 0

    def path_counts(self):
        """Which interchangeable paths this layer's blocks took (infllm_layer_path_counts)."""
        counts = (ctypes.c_int64 * 6)()
        if self._layer:
            check(self._lib.infllm_layer_path_counts(self._layer, counts), "infllm_layer_path_counts")
        return dict(zip(("tables_inline", "tables_kernel", "tables_upload", "score_merged", "score_apart", "call_ranked"),
                        (int(c) for c in counts)))

    def fetched_units(self):
        """Units moved from pinned host memory to the device cache so far (wrongly guessed ones and repairs included)."""
        return int(self._lib.infllm_layer_fetched_units(self._layer)) if self._layer else 0

    def read_timing(self, which):
        """[(ms, n_queries, n_keys)] of the timed launches; which = 0 local stage, 1 global stage."""
        cap = self._timing_cap
        ms, nq, nk = (ctypes.c_float * cap)(), (ctypes.c_int32 * cap)(), (ctypes.c_int32 * cap)()
        n = self._lib.infllm_layer_read_timing(self._layer, which, ms, nq, nk, cap)
        if n < 0:
            check(n, "infllm_layer_read_timing")
        return [(ms[i], nq[i], nk[i]) for i in range(n)]

    # -------------------------------------------------------- one exec block
    def _block(self, st, n, out_ptr, n_next, preselected=None):
        lib, layer, fa, ba = self._lib, self._layer, self._fa, self._ba
        B, bs, topk = self.num_units, self.block_size, self.topk
        b0 = self.length + st
        b1 = b0 + n
        N = self.num_global_block
        fa.d_q = self._q_ptr + st * self._q_step
        fa.d_k = self._k_ptr + st * self._k_step
        fa.d_v = self._v_ptr + st * self._v_step
        fa.n, fa.n_units, fa.b0 = n, N, b0
        fa.n_next = n_next
        fa.flags = ba.flags = _lib.NO_RETRIEVAL if preselected is not None else 0
        if n_next:
            fa.d_q_next = fa.d_q + n * self._q_step
            fa.d_k_next = fa.d_k + n * self._k_step
            fa.d_v_next = fa.d_v + n * self._v_step
        rc = lib.infllm_block_front(layer, self._fa_ref, self._main_raw)
        if rc:
            check(rc, "infllm_block_front")
        # ---- retrieval result (context_manager.py:366-383) -> cache policy (495-515) -> fetch, in one native call:
        #      this stretch is on the chain from one block's selection to the next, the rest of the host's work is not
        sa = self._sa
        stats = self.stats
        if self._mass_units is not None:                     # lru-s: the previous block's masses decide this eviction
            check(lib.infllm_layer_wait_mass(layer), "infllm_layer_wait_mass")
            masses = self.mass_host.tolist()
            for u in range(B):
                self.policy[u].add_scores(self._mass_units[u], masses[u][:len(self._mass_units[u])])
            self._mass_units = None
        # ---- state machine after the block (context_manager.py:614-679): it does not depend on the selection, so the
        #      arguments of the block's second half are ready before the host waits for the ids
        cursor, init_len = self.cursor, self.init_len
        live = b1 - cursor
        take = 0
        if init_len < self.n_init and live > self.n_local:
            take = min(self.n_init - init_len, live - self.n_local)
            live -= take
        c = max((live - self.n_local) // bs, 0)
        ba.n, ba.b0 = n, b0
        ba.init_len, ba.cursor = init_len, cursor
        ba.d_out = out_ptr
        ba.init_take, ba.n_carve, ba.n_units = take, c, N
        idx_out = None
        if c:
            if N + c > self.reps.shape[1]:
                self._grow_reps(N + c)
            ba.d_rep_out = self._reps_ptr + N * self._rep_su_bytes
            for i in range(c):
                self._carve_dst[i] = self._host_unit_addr(N + i)
            if self.record_trace:
                idx_out = torch.empty((B, c, self.unit_size, self.repr_topk), dtype=torch.int32, device=self.device)
            ba.d_repr_idx = idx_out.data_ptr() if idx_out is not None else None
        if self.select_in_steps:
            n_sel, n_miss, selected = self._select_stepwise(preselected, N)
            ba.n_sel, ba.n_miss = n_sel, n_miss
            rc = lib.infllm_block_back(layer, self._ba_ref, self._main_raw, self._copy_raw)
            if rc:
                check(rc, "infllm_block_back")
        else:
            if preselected is not None or N <= topk:
                # chosen for the whole chunk (context_manager.py:381-382), or every unit there is
                selected = preselected if preselected is not None else [list(range(N))] * B
                n_sel = len(selected[0])
                for u in range(B):
                    self._sel_ids[u * n_sel:(u + 1) * n_sel] = selected[u]
                sa.h_selected, sa.n_sel, sa.wait_topk = ctypes.addressof(self._sel_ids), n_sel, 0
            else:
                n_sel = topk
                sa.h_selected, sa.n_sel, sa.wait_topk = self.topk_idx_host.data_ptr(), n_sel, 1   # the one host wait of a block
                selected = None                                   # read back below, off the chain
            ba.n_sel = n_sel
            # selection -> policy -> fetch, then the block's second half at once: next to nothing of the interpreter sits
            # between the arrival of the ids and the launch of the global stage (one native call for both measured no faster)
            n_miss = lib.infllm_block_select(layer, self._sa_ref, self._main_raw, self._copy_raw)
            if n_miss < 0:
                check(n_miss, "infllm_block_select")
            ba.n_miss = n_miss
            rc = lib.infllm_block_back(layer, self._ba_ref, self._main_raw, self._copy_raw)
            if rc:
                check(rc, "infllm_block_back")
            if selected is None and (self.record_trace or self.cache_strategy == "lru-s"):
                # from the library's copy: the pinned ids belong to the next selection once the second half is enqueued
                got = lib.infllm_layer_last_selection(layer, self._sel_ids, len(self._sel_ids))
                if got != B * n_sel:
                    check(min(got, -1), "infllm_layer_last_selection")
                selected = [self._sel_ids[u * n_sel:(u + 1) * n_sel] for u in range(B)]
            stats["evictions"] += sum(self._n_evicted[:B])
            for u in range(B):
                if self.policy[u].evicted_log is not None:
                    self.policy[u].evicted_log.append(list(self._evicted[u * n_sel:u * n_sel + self._n_evicted[u]]))
        stats["hits"] += B * n_sel - n_miss
        stats["misses"] += n_miss
        if self.cache_strategy == "lru":
            self.load_count += 1
        if n_next and preselected is None and self.fetch_ahead and not self.select_in_steps and self.cache_strategy != "lru-s":
            sa.n_sel = topk
            rc = lib.infllm_block_prefetch(layer, self._sa_ref, self._main_raw, self._copy_raw)
            if rc < 0:
                check(rc, "infllm_block_prefetch")
        if self.cache_strategy == "lru-s" and n_sel:
            self._mass_units = selected
        if self.record_trace:
            self.trace_blocks.append(dict(b0=b0, b1=b1, selected=[sorted(s) for s in selected], order=[list(s) for s in selected],
                                          n_units=N, init_len=init_len))
            if c:
                self.trace_units.append((N, c, idx_out))
        stats["blocks"] += 1
        self.init_len = init_len + take
        self.cursor = cursor + take + c * bs
        self.num_global_block = N + c

    def _select_stepwise(self, preselected, N):
        """The same as infllm_block_select in the separate steps the C ABI also offers (a caller with a policy of
        its own would use them): wait for the ids, one infllm_cache_touch per row, build the lists, issue the fetch."""
        lib, layer, B = self._lib, self._layer, self.num_units
        if preselected is not None:
            selected = preselected
        elif N <= self.topk:
            selected = [list(range(N))] * B
        else:
            check(lib.infllm_layer_wait_topk(layer), "infllm_layer_wait_topk")
            selected = self.topk_idx_host.tolist()
        n_sel, n_miss = len(selected[0]), 0
        for u in range(B):
            pol = self.policy[u]
            misses, evicted = pol.touch(selected[u])
            self.stats["evictions"] += len(evicted)
            slot_of = pol.slot_of
            for i, unit in enumerate(selected[u]):
                self._sel_slots[u * n_sel + i] = slot_of[unit]
            for unit in misses:
                chunk, idx = divmod(unit, _HOST_CHUNK_UNITS)
                self._miss_row[n_miss], self._miss_slot[n_miss], self._miss_unit[n_miss] = u, slot_of[unit], unit
                self._miss_src[n_miss] = self._host_dev_base[chunk] + idx * self.unit_bytes + u * self.slot_bytes
                n_miss += 1
        check(lib.infllm_block_fetch(layer, n_miss, self._miss_row, self._miss_slot, self._miss_unit, self._miss_src,
                                     self._main_raw, self._copy_raw), "infllm_block_fetch")
        return n_sel, n_miss, selected

    def _chunk_topk(self, q, c0, c1):
        """Selections of every execution block of q[:, :, c0:c1] against the units that exist now
        (get_batched_topk, context_manager.py:548-612); one host wait for the whole chunk."""
        B, N, topk, exc = self.num_units, self.num_global_block, self.topk, self.exc_block_size
        n_blocks = -(-(c1 - c0) // exc)
        if N <= topk:
            return [[list(range(N))] * B for _ in range(n_blocks)]
        C = self.unit_size * self.head_width
        qbar = torch.empty((B, n_blocks, C), dtype=torch.float32, device=self.device)
        check(self._lib.infllm_chunk_qbar(q.data_ptr() + c0 * q.stride(2) * 2, q.stride(0), q.stride(1), q.stride(2), B,
                                          self.unit_size, c1 - c0, exc, self.inv_freq.data_ptr(),
                                          float(self.position_embedding.distance_scale), self.n_local - 1,
                                          qbar.data_ptr(), self._main_raw), "infllm_chunk_qbar")
        # every block's mean query over the same units: the representatives are read once per eight blocks
        scores = torch.empty((n_blocks, N), dtype=torch.float32, device=self.device)
        idx = torch.empty((n_blocks, B, topk), dtype=torch.int32, device=self.device)
        for u in range(B):
            rc = self._lib.infllm_score_topk_queries(self.reps[u].data_ptr(), self.reps.stride(1), N, C, qbar[u].data_ptr(), qbar.stride(1),
                                                     n_blocks, topk, scores.data_ptr(), scores.stride(0), idx[:, u].data_ptr(),
                                                     idx.stride(0), self._main_raw)
            if rc == 1:                                      # row lengths without that kernel: one block at a time
                for j in range(n_blocks):
                    check(self._lib.infllm_score_topk(self.reps[u].data_ptr(), self.reps.stride(1), N, C, qbar[u, j].data_ptr(),
                                                      topk, scores.data_ptr(), idx[j, u].data_ptr(), self._main_raw),
                          "infllm_score_topk")
            else:
                check(rc, "infllm_score_topk_queries")
        return idx.cpu().tolist()

    def _grow_reps(self, need):
        B, N = self.num_units, self.num_global_block
        rows = max(2 * self.reps.shape[1], need)
        grown = torch.zeros((B, rows, self.reps.shape[2]), dtype=torch.bfloat16, device=self.device)
        grown[:, :N] = self.reps[:, :N]
        scores = torch.empty((B, rows), dtype=torch.float32, device=self.device)
        scores[:, :N] = self.unit_scores[:, :N]          # scores prepared ahead for the next block
        self.reps, self.unit_scores = grown, scores
        self._bind_reps()

    def _bind_reps(self):
        fa, ba = self._fa, self._ba
        self._reps_ptr = self.reps.data_ptr()
        self._rep_su_bytes = self.reps.stride(1) * 2
        fa.d_reps, fa.rep_sb, fa.rep_su = self._reps_ptr, self.reps.stride(0), self.reps.stride(1)
        fa.d_unit_scores, fa.unit_scores_sb = self.unit_scores.data_ptr(), self.unit_scores.stride(0)
        ba.rep_sb, ba.rep_su = self.reps.stride(0), self.reps.stride(1)
        ba.d_reps, ba.d_unit_scores, ba.unit_scores_sb = fa.d_reps, fa.d_unit_scores, fa.unit_scores_sb

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
            self.dim_head = q.size(3)
            check_head_dim(self.dim_head)
        if q.size(3) != self.dim_head:
            raise ValueError(f"head_dim changed from {self.dim_head} to {q.size(3)}")
        q, k, v = _widen(q, self.dim_head), _widen(k, self.dim_head), _widen(v, self.dim_head)
        if not self.initialized:
            self._init(q, k)
            self._bind_reps()
        assert q.shape[:2] == (self.num_units, self.unit_size) and k.shape[1] == self.unit_size_kv

        def rows16(t):          # rows must be contiguous and 16-byte aligned for the vector loads
            ok = t.stride(-1) == 1 and not any(s % 8 for s in t.stride()[:-1]) and t.data_ptr() % 16 == 0
            return t if ok else t.contiguous()
        q, k, v = rows16(q), rows16(k), rows16(v)
        out = torch.empty((self.num_units, self.unit_size, input_length, self.head_width), dtype=torch.bfloat16, device=q.device)
        fa, ba = self._fa, self._ba
        fa.q_sb, fa.q_sh, fa.q_sl = q.stride(0), q.stride(1), q.stride(2)
        fa.k_sb, fa.k_sh, fa.k_sl = k.stride(0), k.stride(1), k.stride(2)
        fa.v_sb, fa.v_sh, fa.v_sl = v.stride(0), v.stride(1), v.stride(2)
        ba.o_sb, ba.o_sh, ba.o_sl = out.stride(0), out.stride(1), out.stride(2)
        self._q_ptr, self._k_ptr, self._v_ptr = q.data_ptr(), k.data_ptr(), v.data_ptr()
        self._q_step, self._k_step, self._v_step = q.stride(2) * 2, k.stride(2) * 2, v.stride(2) * 2
        main = torch.cuda.current_stream()
        self._main_raw = main.cuda_stream
        self._copy_raw = _SIDE_STREAM.cuda_stream if self.async_global_stream else self._main_raw
        if self._call_tokens and self._call_stream != self._main_raw:
            self._bind_call_buffers(self._main_raw)
        out_ptr, out_step = out.data_ptr(), out.stride(2) * 2
        exc = self.exc_block_size
        use_chunks = self.chunk_topk_calc is not None and input_length > 1      # context_manager.py:749-760
        if use_chunks:
            per_chunk = self.chunk_topk_calc // exc
            cuts = [i * exc for i in range(0, input_length // exc + 1, per_chunk)]
            if cuts[-1] < input_length:
                cuts.append(input_length)
            cut_i, plan, plan_pos = -1, None, 0
        call_end = 0
        for st in range(0, input_length, exc):
            n = min(exc, input_length - st)
            if self._call_tokens and st == call_end:
                # the next stretch of the call in one go: prologue, mean queries, first retrieval, local stage
                call_end = min(st + self._call_tokens, input_length)
                if self.length + call_end - self.cursor > self.ring_cap:
                    raise RuntimeError(f"a call of {call_end} tokens at {self.length} does not fit the rings "
                                       f"({self.ring_cap} rows, carving cursor {self.cursor})")
                if call_end - st > exc:          # a single block (a decode step) gains nothing from being prepared apart
                    fa.d_q, fa.d_k, fa.d_v = (self._q_ptr + st * self._q_step, self._k_ptr + st * self._k_step,
                                              self._v_ptr + st * self._v_step)
                    fa.n, fa.n_units, fa.b0 = call_end - st, self.num_global_block, self.length + st
                    fa.flags = _lib.NO_RETRIEVAL if use_chunks else 0
                    # room for every block's scores of the units there are and of those the call can carve
                    blocks, cols = -(-self._call_tokens // exc), self.num_global_block + (call_end - st) // self.block_size + 2
                    if self._call_scores is None or self._call_scores.shape[2] < cols or self._call_scores.shape[0] < blocks:
                        cols = max(-(-cols // 256) * 256, 2 * (self._call_scores.shape[2] if self._call_scores is not None else 0))
                        self._call_scores = torch.empty((blocks, self.num_units, cols), dtype=torch.float32, device=self.device)
                    fa.d_call_scores, fa.call_scores_cols = self._call_scores.data_ptr(), self._call_scores.shape[2]
                    check(self._lib.infllm_call_front(self._layer, self._fa_ref, self._main_raw), "infllm_call_front")
            elif not self._call_tokens:
                call_end = input_length
            chosen = None
            if use_chunks:
                if cuts[cut_i + 1] < st + n:
                    cut_i += 1
                    plan, plan_pos = self._chunk_topk(q, cuts[cut_i], cuts[cut_i + 1]), 0
                chosen = plan[plan_pos]
                plan_pos += 1
            self._block(st, n, out_ptr + st * out_step, min(exc, call_end - st - n), chosen)
        self.length += input_length
        # (the last carved units go on to their pinned home in the background: _finish_host_copies before reading them)
        check(self._lib.infllm_layer_end_call(self._layer, self._copy_raw), "infllm_layer_end_call")
        self._host_copies_open = True
        out = _narrow(out, self.dim_head)
        if self.perhead:
            out = out.view(batch_size, heads, input_length, -1)
        return out

    # ------------------------------------------------------- state in / out
    # The reference keeps its state only in the live object (context_manager.py:292-363); these two
    # methods let a harness start from a prepared memory (e.g. 8192 units with representatives) or resume.
    def export_state(self, with_units=True):
        """Snapshot after an append(): everything a fresh ContextManager needs to continue the stream.
        with_units=False leaves the units out (4 GiB at a million tokens): host_unit(u) still reads them in place."""
        self._finish_host_copies()
        torch.cuda.synchronize()
        T, cur, cap = self.length, self.cursor, self.ring_cap
        rows = torch.arange(cur, T, device=self.device) % cap
        units = [self.host_unit(u).clone() for u in range(self.num_global_block)] if with_units else []
        d, n = self.dim_head, self.num_global_block
        reps = _narrow(self.reps[:, :n].view(self.num_units, n, self.unit_size, self.head_width), d).reshape(self.num_units, n, -1)
        return dict(length=T, n_units=n, init_len=self.init_len,
                    tail_k=_narrow(self.ring_k_raw[:, :, rows], d).clone(), tail_v=_narrow(self.ring_v[:, :, rows], d).clone(),
                    tail_score=self.ring_score[:, :, rows].clone(),
                    init_k=_narrow(self.init_kv[:, 0, :, :self.init_len], d).clone(),
                    init_v=_narrow(self.init_kv[:, 1, :, :self.init_len], d).clone(),
                    units=torch.stack(units) if units else None, reps=reps.clone())

    def load_state(self, state):
        """Start from a prepared memory.  ``state``: length T; tail_k/tail_v [B,Hkv,T-cursor,D] (un-rotated,
        the tokens not carved yet, which include the local window); tail_score [B,H,T-cursor] fp32 or None;
        init_k/init_v [B,Hkv,init_len,D]; units [n_units,B,2,Hkv,bs,D] (any device) or None; reps
        [B,n_units,H*D].  The counts must satisfy the stream's closed forms (context_manager.py:614-679):
        init_len = min(n_init, max(T-n_local, 0)), n_units = max(0, (T-n_init-n_local)//block_size)."""
        from .. import ops
        assert not self.initialized and self.length == 0, "load_state needs a fresh ContextManager"
        tail_k, tail_v = state["tail_k"], state["tail_v"]
        T = int(state["length"])
        B, Hkv, n_tail, D = tail_k.shape
        reps = state["reps"]
        H = reps.shape[2] // D if reps is not None and reps.numel() else state["num_heads"]
        init_len = min(self.n_init, max(T - self.n_local, 0))
        n_units = max(0, (T - self.n_init - self.n_local) // self.block_size)
        cursor = init_len + n_units * self.block_size
        assert n_tail == T - cursor, f"tail holds {n_tail} tokens, the stream state needs {T - cursor}"
        assert state["init_k"].shape[2] == init_len and (n_units == 0 or state["units"].shape[0] == n_units)
        check_head_dim(D)
        self.dim_head = D
        tail_k, tail_v = _widen(tail_k, D), _widen(tail_v, D)
        q_like = torch.empty((B, H, 1, HEAD_DIM), dtype=torch.bfloat16, device=tail_k.device)
        self._init(q_like, tail_k[:, :, :1])
        self._bind_reps()
        self.length, self.cursor, self.init_len = T, cursor, init_len
        if init_len:
            self.init_kv[:, 0, :, :init_len] = _widen(state["init_k"], D)
            self.init_kv[:, 1, :, :init_len] = _widen(state["init_v"], D)
        if n_units:
            self._grow_reps(n_units) if n_units > self.reps.shape[1] else None
            self.reps[:, :n_units] = _widen(reps.view(B, n_units, H, D), D).reshape(B, n_units, -1)
            for u in range(n_units):
                self._host_unit_addr(u)                        # allocates the pinned chunk
                self._host_unit_rows(u).copy_(_widen(state["units"][u], D))
            self.num_global_block = n_units
        # tail -> rings (RoPE at the absolute positions) in pieces of one execution block
        D = HEAD_DIM
        zq = torch.zeros((B, H, self.exc_block_size, D), dtype=torch.bfloat16, device=self.device)
        for st in range(0, n_tail, self.exc_block_size):
            n = min(self.exc_block_size, n_tail - st)
            ops.ingest(zq[:, :, :n], tail_k[:, :, st:st + n], tail_v[:, :, st:st + n], cursor + st, self.n_local - 1,
                       self.inv_freq, float(self.position_embedding.distance_scale), self.ring_k_raw, self.ring_k_rot,
                       self.ring_v, self.ring_score, self.q_loc[0], self.q_glb[0])
        if state.get("tail_score") is not None:
            rows = torch.arange(cursor, T, device=self.device) % self.ring_cap
            self.ring_score[:, :, rows] = state["tail_score"].to(torch.float32)
        torch.cuda.synchronize()
        return self

    # ----------------------------------------------------------------- tracing
    def trace_repr_indices(self):
        """{unit: int tensor [B, H, repr_topk]} of the keys chosen as representatives (needs record_trace)."""
        res = {}
        for first, count, idx in self.trace_units:
            host = idx.cpu()
            for i in range(count):
                res[first + i] = host[:, i]
        return res
