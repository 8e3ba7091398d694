"""Throughput of the InfLLM streaming memory-attention path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

One step = one pass of a single attention layer (Mistral-7B geometry: 32 query
heads, 8 kv heads, head_dim 128, RoPE base 1e6) over a 131,072-token synthetic
stream, consumed in execution blocks of 512 tokens with the reference's default
knobs (n_init 128, n_local 4096, block 128, topk 16, repr_topk 4,
max_cached_block 32, lru).  Inputs are resident in HBM before the timed region.
Prints ONE JSON line with tokens/s, the roofline of the dominant kernel (the
MFMA attention stage, timed with events on its own stream during the timed
steps) and the CPU baseline (the fp32 oracle on a bounded sample, host cores).
"""
import argparse
import json
import os
import sys
import time

import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

H, HKV, D = 32, 8, 128
KNOBS = dict(n_init=128, n_local=4096, block_size=128, max_cached_block=32, topk=16, exc_block_size=512, repr_topk=4)
ROPE_BASE = 1e6
MFMA_BF16_PEAK_TFLOPS = 2500.0


def make_stream(T, seed, device, favour=0):
    """q, v ~ N(0,1); keys from a 64-component Gaussian mixture per kv head (means N(0,1), std 0.3).
    favour > 0 (benchmark configuration 5): the queries of an execution block lean towards `favour` mixture components
    drawn per block (q = that component's mean + N(0,1)), so consecutive blocks retrieve different units."""
    g = torch.Generator(device=device).manual_seed(seed)
    means = torch.randn((HKV, 64, D), generator=g, device=device)
    q = torch.empty((1, H, T, D), dtype=torch.bfloat16, device=device)
    k = torch.empty((1, HKV, T, D), dtype=torch.bfloat16, device=device)
    v = torch.empty((1, HKV, T, D), dtype=torch.bfloat16, device=device)
    exc = KNOBS["exc_block_size"]
    for t0 in range(0, T, 1 << 17):                     # in slices: the fp32 temporaries of a 1M-token stream are large
        n = min(1 << 17, T - t0)
        qs = torch.randn((H, n, D), generator=g, device=device)
        if favour:
            blocks = (n + exc - 1) // exc
            pick = torch.randint(0, 64, (blocks, favour), generator=g, device=device)
            which = torch.randint(0, favour, (n,), generator=g, device=device)
            comp_q = pick[torch.arange(n, device=device) // exc, which]                      # [n]
            qs += means[:, comp_q].repeat_interleave(H // HKV, dim=0)                         # [H, n, D]
        q[0, :, t0:t0 + n] = qs.bfloat16()
        v[0, :, t0:t0 + n] = torch.randn((HKV, n, D), generator=g, device=device).bfloat16()
        comp = torch.randint(0, 64, (HKV, n), generator=g, device=device)
        ks = torch.gather(means, 1, comp[:, :, None].expand(-1, -1, D)) + 0.3 * torch.randn((HKV, n, D), generator=g, device=device)
        k[0, :, t0:t0 + n] = ks.bfloat16()
    return q, k, v


TIMING_STRIDE = 17          # co-prime with the 16 blocks of an append call: the sample covers every position in a call


def run_stream(q, k, v, chunk, timing=False):
    from infllm_amd.attention import ContextManager, RotaryEmbeddingESM
    rope = RotaryEmbeddingESM(D, base=ROPE_BASE, device=q.device)
    cm = ContextManager(rope, KNOBS["n_init"], KNOBS["n_local"], KNOBS["block_size"], KNOBS["max_cached_block"],
                        KNOBS["topk"], KNOBS["exc_block_size"], None, True, KNOBS["repr_topk"], "lru", None, True, True)
    T = q.shape[2]
    if timing:
        # an event pair around a launch costs the stream several microseconds (5% of the stream when every attention
        # launch carries one), so the timed region samples every TIMING_STRIDE-th launch of each stage
        cm.enable_timing(T // KNOBS["exc_block_size"] // TIMING_STRIDE + 2, TIMING_STRIDE)
    out = None
    for st in range(0, T, chunk):
        sl = slice(st, min(st + chunk, T))
        out = cm.append(q[:, :, sl], k[:, :, sl], v[:, :, sl], q[:, :, sl], k[:, :, sl], v[:, :, sl])
    return cm, out


def counted_traffic(summary, key):
    """HBM bytes per launch from hardware counters (FETCH_SIZE, WRITE_SIZE; one profiler run per counter, each scaled
    by what the counter reads for a 256 MiB elementwise pass).  The figure is not measured in this run: it is read from
    the rocprofv3 summary under profiles/ that derives it, which carries a line `<key> = <bytes>`; None when the
    summary is not there (the figures hold for the default geometry only)."""
    import re
    try:
        with open(os.path.join(ROOT, "profiles", summary)) as f:
            m = re.search(r"^%s\s*=\s*(\d+)" % re.escape(key), f.read(), re.M)
        return int(m.group(1)) if m else None
    except OSError:
        return None


def _event_time_us(fn, launches, warm):
    """mean microseconds per call of fn(i), timed with events on the stream the kernels are launched on"""
    for i in range(warm):
        fn(i)
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for i in range(launches):
        fn(i)
    e1.record()
    torch.cuda.synchronize()
    return e0.elapsed_time(e1) / launches * 1e3


def _hbm_entry(kernel, what, nbytes, us, launches, **extra):
    gbs = nbytes / (us * 1e-6) / 1e9
    return dict(kernel=kernel, what=what, algorithmic_bytes=int(nbytes), avg_us=us, GBps=gbs, frac_of_8TBps=gbs / 8000.0,
                launches_timed=launches, **extra)


def hbm_leg(dev, n_units=8192, tables=8, launches=200):
    """The HBM half of the metric, measured in this run: a RETRIEVAL (context_manager.py:159-163: unit scores, then
    their top-k) over n_units representatives of H*D bf16 each, the shape of benchmark configuration 3, as ONE launch -
    N*H*D*2 algorithmic bytes (64 MiB), read once (the selection re-reads the N fp32 scores: 32 KiB).  The launches
    rotate over `tables` distinct tables (512 MiB together, more than the 256 MB of last-level cache), so every launch
    reads from HBM; the figure is the MEAN over all launches, timed with events on the stream the kernel runs on.
    Returns (roofline object of the retrieval, entry of the scoring kernel alone)."""
    from infllm_amd import ops
    C, k = H * D, KNOBS["topk"]
    reps = torch.randn((tables, n_units, C), device=dev, dtype=torch.bfloat16)
    qbar = torch.randn((C,), device=dev)
    scores = torch.empty((n_units,), dtype=torch.float32, device=dev)
    idx = torch.empty((k,), dtype=torch.int32, device=dev)
    nbytes = n_units * C * 2
    us = _event_time_us(lambda i: ops.score_topk(reps[i % tables], n_units, qbar, k, scores, idx), launches, 2 * tables)
    gbs = nbytes / (us * 1e-6) / 1e9
    retrieval = {"bound": "hbm", "achieved": gbs, "peak": 8000.0, "unit": "GB/s", "frac": gbs / 8000.0,
                 "traffic": counted_traffic("retrieval__decode8192.hbm_bytes.txt", "retrieval_traffic_bytes"),
                 "kernel": f"retrieve_fused_kernel<8, 2>: unit scores + top-{k} in one launch ({n_units} x {C} bf16 representatives = "
                           f"{nbytes / 2 ** 20:.0f} MiB per launch, {tables} tables in rotation)",
                 "avg_launch_ms": us * 1e-3, "launches_timed": launches}
    us = _event_time_us(lambda i: ops.score_topk(reps[i % tables], n_units, qbar, 0, scores, None), launches, 2 * tables)
    scoring = _hbm_entry("unit_scores_rows_kernel<8, 2>", f"unit scores alone, {n_units} x {C} bf16, {tables} tables in rotation", nbytes, us,
                         launches, traffic=counted_traffic("retrieval__decode8192.hbm_bytes.txt", "unit_scores_traffic_bytes"))
    return retrieval, scoring


def call_lists_entry(dev, n_units=8192, tables=8, queries=15, launches=40):
    """The lists of a prepared call (infllm_score_topk_queries): the scores of n_units representatives under the mean queries
    of a call's other 15 blocks and the 16 best per query, the representatives read once per eight queries.  Algorithmic
    bytes: the representatives once (N*H*D*2) plus the queries' score rows written and read by the selection."""
    from infllm_amd import ops
    C, k = H * D, KNOBS["topk"]
    reps = torch.randn((tables, n_units, C), device=dev, dtype=torch.bfloat16)
    qbars = torch.randn((queries, C), device=dev)
    scores = torch.empty((queries, n_units), dtype=torch.float32, device=dev)
    idx = torch.empty((queries, k), dtype=torch.int32, device=dev)
    us = _event_time_us(lambda i: ops.score_topk_queries(reps[i % tables], n_units, qbars, k, scores, idx), launches, 2 * tables)
    nbytes = n_units * C * 2 + 2 * queries * n_units * 4
    return _hbm_entry("unit_scores_queries_kernel<8> + select_rows_kernel<1>",
                      f"lists of a call: {queries} mean queries over {n_units} x {C} bf16 representatives, top-{k} each, two launches "
                      f"({tables} tables in rotation; the same by one retrieval per block: {queries} x {n_units * C * 2 / 2 ** 20:.0f} MiB)",
                      nbytes, us, launches)


def kernels_hbm_leg(dev):
    """The other HBM-bound kernels of the path at the shapes the benchmark configurations give them, each timed in this
    run with events over repeated launches; algorithmic bytes as the scope table counts them.  Inputs of more than a
    few MB rotate over enough copies to exceed the last-level cache."""
    import ctypes
    from infllm_amd import ops
    out = []
    bf = dict(dtype=torch.bfloat16, device=dev)
    n_local, bs, n_init, topk, exc = (KNOBS[k] for k in ("n_local", "block_size", "n_init", "topk", "exc_block_size"))
    # ---- prologue of an append() call: RoPE, rings, rotated queries (rope.py:4-112, context_manager.py:712-747)
    n = 8192
    cap = (n_local + exc + bs + n + 63) // 64 * 64 + 64
    q, k, v = (torch.randn((1, h, n, D), device=dev).bfloat16() for h in (H, HKV, HKV))
    rings = [torch.zeros((1, HKV, cap, D), **bf) for _ in range(3)]
    ring_score = torch.zeros((1, H, cap), dtype=torch.float32, device=dev)
    q_loc, q_glb = torch.empty((1, H, n, D), **bf), torch.empty((1, H, n, D), **bf)
    qpart = torch.empty((1, (n + 15) // 16, H * D), dtype=torch.float32, device=dev)
    inv_freq = (ROPE_BASE ** (-torch.arange(0, D, 2, dtype=torch.float32) / D)).to(dev)
    us = _event_time_us(lambda i: ops.ingest(q, k, v, 100000 + i * n, n_local - 1, inv_freq, 1.0, *rings, ring_score, q_loc, q_glb, qpart), 20, 3)
    per_token = (H + 2 * HKV) * D * 2 + 2 * H * D * 2 + 3 * HKV * D * 2
    out.append(_hbm_entry("ingest_kernel", f"prologue of an {n}-token append() call: reads q, k, v, writes both rotated q and three ring rows "
                                           f"({per_token} B per token)", n * per_token, us, 20,
                          traffic=counted_traffic("retrieval__decode8192.hbm_bytes.txt", "ingest_traffic_bytes")))
    del q, k, v, q_loc, q_glb, qpart
    # ---- representatives of the units a block carves (context_manager.py:268-277) and their rows out of the rings
    n_units = exc // bs
    rs = torch.rand((1, H, cap), dtype=torch.float32, device=dev)
    rep = torch.empty((1, 64, H * D), **bf)
    us = _event_time_us(lambda i: ops.repr_keys(rs, rings[0], 5000 + 7 * i, bs, n_units, KNOBS["repr_topk"], rep, rep.stride(0), rep.stride(1)), 200, 10)
    per_unit = H * bs * 4 + H * KNOBS["repr_topk"] * D * 2 + H * D * 2
    out.append(_hbm_entry("repr_keys_kernel", f"representatives of the {n_units} units of a block: scores, {KNOBS['repr_topk']} gathered keys per head, "
                                              f"one row out ({per_unit} B per unit); a chain of dependent arg-max steps, latency-bound",
                          n_units * per_unit, us, 200, traffic=counted_traffic("retrieval__decode8192.hbm_bytes.txt", "repr_keys_traffic_bytes")))
    stage = torch.empty((n_units, 1, 2, HKV, bs, D), **bf)

    def gather(i):
        for which, ring in ((0, rings[0]), (1, rings[2])):
            ops.gather_rows(ring, 5000 + 7 * i, n_units * bs, stage[0, 0, which].data_ptr(), stage.stride(1), stage.stride(3),
                            unit_rows=bs, out_su=stage.stride(0))
    unit_bytes = 2 * HKV * bs * D * 2
    us = _event_time_us(gather, 200, 10)
    out.append(_hbm_entry("gather_rows_kernel x2", f"K and V rows of a block's {n_units} carved units, ring -> staging ({unit_bytes} B per unit, "
                                                   "read and written once; two launches of 3 us whose event-timed mean is mostly launch gap; in the stream "
                                                   "this copy rides in the repr_keys launch)", n_units * unit_bytes, us, 200,
                          traffic=counted_traffic("retrieval__decode8192.hbm_bytes.txt", "gather_rows_traffic_bytes")))
    # ---- decode-shaped attention (config 3): one query per head over the window and the retrieved units, both stages + merge
    sets, n_glob = 12, topk * bs + n_init + 64
    ns_l, ns_g = 32, (n_glob // 64) // 2
    capd = (n_local + 64 + 63) // 64 * 64 + 64
    qd = torch.randn((1, H, 1, D), device=dev).bfloat16()
    ring_k, ring_v = torch.randn((sets, 1, HKV, capd, D), device=dev).bfloat16(), torch.randn((sets, 1, HKV, capd, D), device=dev).bfloat16()
    pool = torch.randn((sets, 2, HKV, n_glob, D), device=dev).bfloat16()
    n_pages = n_glob // 64
    pages = []
    for s_ in range(sets):
        ent = [(pool[s_, 0].data_ptr() + i * 64 * D * 2, pool[s_, 1].data_ptr() + i * 64 * D * 2, n_glob * D, 64) for i in range(n_pages)]
        arr = ops.make_pages(ent)
        host = torch.empty((n_pages * 32,), dtype=torch.uint8)
        ctypes.memmove(host.data_ptr(), arr, n_pages * 32)
        pages.append(host.to(dev))
    o_part = torch.empty((ns_l + ns_g, 1, H, 1, D), dtype=torch.float16, device=dev)
    lse_part = torch.empty((ns_l + ns_g, 1, H, 1), dtype=torch.float32, device=dev)
    o, lse = torch.empty((1, H, 1, D), **bf), torch.empty((1, H, 1), dtype=torch.float32, device=dev)
    b0 = 100000

    def decode_attn(i):
        s_ = i % sets
        la = ops.linear_stage_args(qd, ring_k[s_], ring_v[s_], o_part[:ns_l], lse_part[:ns_l], cap=capd, j_lo=b0 - n_local, j_hi=b0 + 1,
                                   mask=ops.MASK_WINDOW, offset=b0, window=n_local, nsplit=ns_l)
        ga = ops.paged_stage_args(qd, pages[s_], n_pages, HKV, o_part[ns_l:], lse_part[ns_l:], nsplit=ns_g)
        ops.attn_fwd(la, ga, o, lse)
    us = _event_time_us(decode_attn, 200, 2 * sets)
    nbytes = (n_local + 1 + n_glob) * HKV * D * 2 * 2
    out.append(_hbm_entry("attn_stage_kernel<0> + <1> + attn_merge_wide_kernel", f"decode-shaped attention: 1 query x {H} heads over {n_local + 1} window keys "
                          f"({ns_l} key splits) and {n_glob} retrieved keys ({ns_g} splits), K and V read once, three launches; "
                          f"{sets} K/V sets in rotation", nbytes, us, 200,
                          traffic=counted_traffic("retrieval__decode8192.hbm_bytes.txt", "decode_attention_traffic_bytes")))
    return out


def make_decode_state(dev, n_units, seed=3):
    """A prepared memory for the decode shape (benchmark configuration 3): n_units units of mixture keys with representatives
    (the mean of each unit's first repr_topk keys), a full local window and the init tokens.  Returns the state
    ContextManager.load_state takes, and a function drawing further (q, k, v) tokens from the same generator."""
    bs, n_local, n_init = KNOBS["block_size"], KNOBS["n_local"], KNOBS["n_init"]
    T0 = n_init + n_units * bs + n_local
    g = torch.Generator(device=dev).manual_seed(seed)
    means = torch.randn((HKV, 64, D), generator=g, device=dev)

    def mixture_keys(n):
        comp = torch.randint(0, 64, (HKV, n), generator=g, device=dev)
        k = torch.gather(means, 1, comp[:, :, None].expand(-1, -1, D)) + 0.3 * torch.randn((HKV, n, D), generator=g, device=dev)
        return k[None].bfloat16()

    units = torch.empty((n_units, 1, 2, HKV, bs, D), dtype=torch.bfloat16, device=dev)
    reps = torch.empty((1, n_units, H * D), dtype=torch.bfloat16, device=dev)
    for u0 in range(0, n_units, 512):                      # built in slices to bound temporary memory
        n = min(512, n_units - u0)
        k = mixture_keys(n * bs)[0].view(HKV, n, bs, D)
        units[u0:u0 + n, 0, 0] = k.permute(1, 0, 2, 3)
        units[u0:u0 + n, 0, 1] = torch.randn((n, HKV, bs, D), generator=g, device=dev).bfloat16()
        rep = k[:, :, :KNOBS["repr_topk"]].float().mean(dim=2)                    # [Hkv, n, D]: mean of 4 keys of the unit
        reps[0, u0:u0 + n] = rep.permute(1, 0, 2).repeat_interleave(H // HKV, dim=1).reshape(n, H * D).bfloat16()
    state = dict(length=T0, tail_k=mixture_keys(n_local), tail_v=torch.randn((1, HKV, n_local, D), generator=g, device=dev).bfloat16(),
                 tail_score=None, init_k=mixture_keys(n_init), init_v=torch.randn((1, HKV, n_init, D), generator=g, device=dev).bfloat16(),
                 units=units, reps=reps)

    def tokens(n):
        q = torch.randn((1, H, n, D), generator=g, device=dev).bfloat16()
        return q, mixture_keys(n), torch.randn((1, HKV, n, D), generator=g, device=dev).bfloat16()

    return state, tokens


def decode_workload(args, dev):
    """benchmark configuration 3: 256 single-token steps over a prepared memory of 8192 units (1,048,576 past tokens)
    with precomputed representatives.  Prints its own JSON line; not the headline metric."""
    from infllm_amd import ops
    from infllm_amd.attention import ContextManager, RotaryEmbeddingESM
    n_units, bs, n_local, n_init, topk = args.decode_units, KNOBS["block_size"], KNOBS["n_local"], KNOBS["n_init"], KNOBS["topk"]
    state, tokens = make_decode_state(dev, n_units)
    rope = RotaryEmbeddingESM(D, base=ROPE_BASE, device=dev)
    cm = ContextManager(rope, n_init, n_local, bs, KNOBS["max_cached_block"], topk, KNOBS["exc_block_size"], None, True,
                        KNOBS["repr_topk"], "lru", None, True, True).load_state(state)
    del state
    steps = args.decode_steps
    q, k, v = tokens(steps + 8)
    for i in range(8):                                      # warm-up steps
        cm.append(q[:, :, i:i + 1], k[:, :, i:i + 1], v[:, :, i:i + 1], q[:, :, i:i + 1], k[:, :, i:i + 1], v[:, :, i:i + 1])
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(8, 8 + steps):
        out = cm.append(q[:, :, i:i + 1], k[:, :, i:i + 1], v[:, :, i:i + 1], q[:, :, i:i + 1], k[:, :, i:i + 1], v[:, :, i:i + 1])
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    assert torch.isfinite(out.float()).all()
    # the HBM-bound kernel of this shape: unit scoring (N x 4096 bf16 representatives read once) + top-k
    N = cm.num_global_block
    scores = torch.empty((N,), dtype=torch.float32, device=dev)
    idx = torch.empty((topk,), dtype=torch.int32, device=dev)
    qbar = torch.randn((H * D,), device=dev)
    for _ in range(5):
        ops.score_topk(cm.reps[0], N, qbar, topk, scores, idx)
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(50):
        ops.score_topk(cm.reps[0], N, qbar, 0, scores, None)
    e1.record()
    torch.cuda.synchronize()
    ms = e0.elapsed_time(e1) / 50
    gbs = N * H * D * 2 / (ms * 1e-3) / 1e9
    print(json.dumps({
        "metric": "InfLLM decode steps/s over a 1M-token memory (1 layer, Mistral-7B geom)", "value": steps / dt, "unit": "tokens/s",
        "n_gpus": 1, "steps": steps, "ms_per_step": dt / steps * 1e3, "higher_is_better": True, "dtype": "bf16", "data": "synthetic",
        "config": {"workload": f"config 3: {steps} single-token steps, {N} units x {bs} tokens, topk {topk}, n_local {n_local}, "
                               f"max_cached {KNOBS['max_cached_block']}"},
        "roofline": {"bound": "hbm", "achieved": gbs, "peak": 8000.0, "unit": "GB/s", "frac": gbs / 8000.0,
                     "traffic": counted_traffic("retrieval__decode8192.hbm_bytes.txt", "unit_scores_traffic_bytes"),
                     "kernel": f"unit_scores_kernel ({N} x {H * D} bf16 representatives, {N * H * D * 2 / 2 ** 20:.1f} MiB per retrieval)",
                     "avg_launch_ms": ms},
        "cache": cm.stats}))


def model_workload(args, dev):
    """benchmark configuration 4: a 32-layer decoder with the Llama-3-8B architecture and random weights, every attention
    routed through the "inf-llm" type; chunked prefill (all but the last token in pieces of 8192, then the last
    token) followed by greedy decode steps, driven by GreedySearch.  Prints its own JSON line; not the headline."""
    import transformers
    from infllm_amd.utils import GreedySearch, patch_hf
    cfg = transformers.LlamaConfig(hidden_size=4096, intermediate_size=14336, num_hidden_layers=args.model_layers,
                                   num_attention_heads=32, num_key_value_heads=8, head_dim=128, vocab_size=128256,
                                   rope_theta=500000.0, max_position_embeddings=8192, tie_word_embeddings=False)
    torch.manual_seed(4)
    old = torch.get_default_dtype()
    torch.set_default_dtype(torch.bfloat16)
    try:
        with torch.device(dev):
            model = transformers.LlamaForCausalLM(cfg)
    finally:
        torch.set_default_dtype(old)
    knobs = {k: KNOBS[k] for k in ("n_init", "n_local", "topk", "block_size", "max_cached_block", "exc_block_size", "repr_topk")}
    model = patch_hf(model, "inf-llm", dict(knobs, fattn=False), base=500000.0).eval()

    class Tok:                                      # token ids in, token ids out
        eos_token_id = -1

        def decode(self, ids):
            return ids.tolist()

    T, steps = args.model_tokens, args.model_decode_steps
    ids = torch.randint(0, 128256, (T,), generator=torch.Generator().manual_seed(5))
    gs = GreedySearch(model, Tok())
    # time the prefill and the decode separately: a first generate() with no new token, then one more that decodes
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    first = gs.generate(input_ids=ids, max_length=0, chunk_size=8192)
    torch.cuda.synchronize()
    t1 = time.perf_counter()
    # the cache now holds the whole prompt; feed the token the prefill chose and keep decoding greedily
    with torch.inference_mode():
        logits, past = gs._step(ids[None, -1:].to(dev), torch.ones((1, T + 1), dtype=torch.long, device=dev), gs.past_kv)
        word = logits[:, -1].argmax(dim=-1)
        torch.cuda.synchronize()
        t2 = time.perf_counter()
        for _ in range(steps):
            logits, past = gs._step(word.view(1, 1), torch.ones((1, 1), dtype=torch.long, device=dev), past)
            word = logits[:, -1].argmax(dim=-1)
        torch.cuda.synchronize()
        t3 = time.perf_counter()
    cm = past[0]
    print(json.dumps({
        "metric": "InfLLM full decoder (Llama-3-8B architecture, random weights): prefill tokens/s", "value": T / (t1 - t0),
        "unit": "tokens/s", "n_gpus": 1, "higher_is_better": True, "dtype": "bf16", "data": "synthetic",
        "config": {"workload": f"config 4: {args.model_layers} layers, {T}-token prefill in chunks of 8192 + last token, "
                               f"then {steps} greedy steps; inf-llm knobs {knobs}"},
        "prefill_s": t1 - t0, "decode_steps_per_s": steps / (t3 - t2), "decode_ms_per_step": (t3 - t2) / steps * 1e3,
        "layer0_cache": cm.stats, "layer0_units": cm.num_global_block}))


def extra_legs(args, dev):
    """The other single-layer configurations, timed in this run so that their figures come with the headline:
    the same 131,072-token stream with every unit resident (nothing crosses PCIe: the kernels' own time), benchmark
    configuration 3 (single-token steps over 8,192 prepared units) and config 5 (one 1,048,576-token stream whose queries
    favour two mixture components per block)."""
    from infllm_amd.attention import ContextManager, RotaryEmbeddingESM
    legs = {}
    keep = KNOBS["max_cached_block"]
    try:
        q, k, v = make_stream(131072, 0, dev)
        KNOBS["max_cached_block"] = 1024

        times, prev = [], None
        for i in range(5):                  # two warm-up steps, three timed ones, each on its own clock
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            cm, _ = run_stream(q, k, v, args.chunk)
            torch.cuda.synchronize()
            times.append(time.perf_counter() - t0)
            prev = cm                       # the previous step's manager goes once this step is done
        del prev, cm
        legs["all_resident_ms_per_step"] = sum(times[2:]) / 3 * 1e3
        del q, k, v
    except Exception as e:                                    # a leg never takes the headline down
        legs["all_resident_ms_per_step"] = {"error": repr(e)}
    finally:
        KNOBS["max_cached_block"] = keep
    try:
        n_units, steps, warm = 8192, 64, 8
        state, tokens = make_decode_state(dev, n_units)
        rope = RotaryEmbeddingESM(D, base=ROPE_BASE, device=dev)
        cm = ContextManager(rope, KNOBS["n_init"], KNOBS["n_local"], KNOBS["block_size"], KNOBS["max_cached_block"], KNOBS["topk"],
                            KNOBS["exc_block_size"], None, True, KNOBS["repr_topk"], "lru", None, True, True).load_state(state)
        del state
        q, k, v = tokens(steps + warm)
        one = lambda i: cm.append(q[:, :, i:i + 1], k[:, :, i:i + 1], v[:, :, i:i + 1], q[:, :, i:i + 1], k[:, :, i:i + 1], v[:, :, i:i + 1])
        for i in range(warm):
            one(i)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for i in range(warm, warm + steps):
            out = one(i)
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
        assert torch.isfinite(out.float()).all()
        legs["decode_leg"] = {"workload": f"config 3: {steps} single-token steps over {n_units} prepared units ({n_units * KNOBS['block_size']} past tokens)",
                              "ms_per_step": dt / steps * 1e3, "steps_per_s": steps / dt, "cache": dict(cm.stats)}
        del cm, q, k, v
    except Exception as e:
        legs["decode_leg"] = {"error": repr(e)}
    try:
        T5 = 1 << 20
        q, k, v = make_stream(T5, 5, dev, favour=2)
        cm, out = run_stream(q, k, v, args.chunk)              # pins the units' host memory once (4 GiB)
        torch.cuda.synchronize()
        del cm, out
        t0 = time.perf_counter()
        cm, out = run_stream(q, k, v, args.chunk)
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
        assert torch.isfinite(out.float()).all() and cm.length == T5
        legs["million_leg"] = {"workload": f"config 5: one {T5}-token stream, queries favour 2 mixture components per block, max_cached {keep}, lru",
                               "ms_per_step": dt * 1e3, "tokens_per_s": T5 / dt, "units": cm.num_global_block, "cache": dict(cm.stats)}
        del cm, q, k, v
    except Exception as e:
        legs["million_leg"] = {"error": repr(e)}
    return legs


def cpu_baseline(tokens, threads, seed=1):
    """benchmark configuration 1: the reference's torch path restated (the fp32 oracle; the reference's own files hard-code
    "cuda") on the host cores - q, k, v i.i.d. N(0,1) from `seed`, fp32, the first `tokens` tokens of the
    16,384-token stream (all of it by default)."""
    from oracle.rope import RopeOracle
    from oracle.stream import StreamOracle
    torch.set_num_threads(threads)
    g = torch.Generator().manual_seed(seed)
    q = torch.randn((1, H, tokens, D), generator=g)
    k = torch.randn((1, HKV, tokens, D), generator=g)
    v = torch.randn((1, HKV, tokens, D), generator=g)
    ora = StreamOracle(RopeOracle(D, base=ROPE_BASE), KNOBS["n_init"], KNOBS["n_local"], KNOBS["block_size"],
                       32, KNOBS["topk"], KNOBS["exc_block_size"], repr_topk=KNOBS["repr_topk"])
    t0 = time.perf_counter()
    ora.append(q, k, v)
    dt = time.perf_counter() - t0
    return dict(value=tokens / dt, unit="tokens/s", cores=threads, kind="port",
                sample=f"config 1: {tokens} of 16384 tokens, q/k/v i.i.d. N(0,1) (torch.Generator seed {seed}), fp32, one append() call, "
                       f"{dt:.1f} s")


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=5)
    ap.add_argument("--warmup", type=int, default=4)
    ap.add_argument("--tokens", type=int, default=131072)
    ap.add_argument("--chunk", type=int, default=8192, help="tokens per append() call")
    ap.add_argument("--cpu-tokens", type=int, default=16384, help="tokens of config 1 the CPU baseline runs (0 disables it)")
    ap.add_argument("--no-hbm-leg", action="store_true", help="skip the HBM-bound kernels' measurements (roofline_hbm, kernels_hbm)")
    ap.add_argument("--no-extra-legs", action="store_true", help="skip the all-resident, decode (config 3) and 1M-token (config 5) legs")
    ap.add_argument("--workload", choices=["prefill", "decode", "model", "hbm"], default="prefill",
                    help="prefill = the headline 128K-token stream (config 2); decode = config 3, model = config 4, "
                         "hbm = the HBM-bound kernels' legs alone (each with its own JSON line)")
    ap.add_argument("--model-layers", type=int, default=32)
    ap.add_argument("--model-tokens", type=int, default=131072)
    ap.add_argument("--model-decode-steps", type=int, default=128)
    ap.add_argument("--decode-units", type=int, default=8192)
    ap.add_argument("--decode-steps", type=int, default=256)
    ap.add_argument("--favour", type=int, default=0,
                    help="queries of a block lean towards this many mixture components (config 5 uses 2 with --tokens 1048576)")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="first run three elementwise passes over 256 MiB (reads 256 MiB, writes 256 MiB each): the known-size "
                         "kernel that hardware byte counters of a profiled run are scaled by")
    ap.add_argument("--max-cached-block", type=int, default=KNOBS["max_cached_block"],
                    help="GPU unit-cache slots (the headline number uses the reference's 32)")
    args = ap.parse_args()
    KNOBS["max_cached_block"] = args.max_cached_block
    if args.gpus != 1:
        sys.exit("bench.py: this build runs on ONE GPU (the path has no cross-GPU step); use --gpus 1")
    assert torch.cuda.is_available(), "bench.py needs a GPU"
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    if args.copy_calibration:
        src = torch.ones((128 << 20,), dtype=torch.bfloat16, device=dev)
        dst = torch.empty_like(src)
        for _ in range(3):
            torch.neg(src, out=dst)
        torch.cuda.synchronize()
        del src, dst
    if args.workload == "decode":
        decode_workload(args, dev)
        return
    if args.workload == "model":
        model_workload(args, dev)
        return
    if args.workload == "hbm":
        retrieval, scoring = hbm_leg(dev)
        print(json.dumps({"roofline_hbm": retrieval, "kernels_hbm": [scoring, call_lists_entry(dev)] + kernels_hbm_leg(dev)}))
        return
    T = args.tokens
    q, k, v = make_stream(T, 0, dev, args.favour)
    torch.cuda.synchronize()

    # A step's manager (pinned home of the units, event timers) is read out and dropped once the NEXT step has been
    # issued: its launches have finished by then (the host follows the stream's selections), and the allocators hand
    # its buffers to the step after - the warm-up steps run the same way, so no timed step allocates pinned memory.
    def run_steps(n):
        records, prev, out = [], None, None
        for _ in range(n):
            cm, out = run_stream(q, k, v, args.chunk, timing=True)
            if prev is not None:
                records.append((prev.read_timing(0), prev.read_timing(1), prev.read_timing(2), prev.prefetch_stats(), dict(prev.stats), (prev.fetched_units(), prev.staged_units())))
            prev = cm
        torch.cuda.synchronize()
        records.append((prev.read_timing(0), prev.read_timing(1), prev.read_timing(2), prev.prefetch_stats(), dict(prev.stats), (prev.fetched_units(), prev.staged_units())))
        return records, out

    run_steps(args.warmup) if args.warmup > 0 else None
    torch.cuda.synchronize()
    # The warm-up goes on, one synchronised step at a time, until three steps in a row are within 8 % of the fastest
    # seen (at most 40 more): a process that starts right after another one has released tens of GB of pinned and
    # device memory can run its first second at two thirds of the speed.  Three steps when there is nothing to wait for.
    settle_ms = []
    while args.warmup > 0 and len(settle_ms) < 40:
        t0 = time.perf_counter()
        run_steps(1)
        settle_ms.append((time.perf_counter() - t0) * 1e3)
        if len(settle_ms) >= 3 and max(settle_ms[-3:]) <= 1.08 * min(settle_ms):
            break
    t0 = time.perf_counter()
    runs, out = run_steps(args.steps)
    dt = time.perf_counter() - t0
    assert torch.isfinite(out.float()).all()
    cm_stats = runs[-1][4]

    # dominant kernel: the local (sliding-window) attention stage; steady-state launches only
    exc, n_local = KNOBS["exc_block_size"], KNOBS["n_local"]
    # (one launch covers every block of an append() call: its queries are the call's, each seeing n_local keys)
    q_launch = max([nq for r in runs for ms, nq, nk in r[0]] or [exc])
    steady = [ms for r in runs for ms, nq, nk in r[0] if nq == q_launch and nk == n_local + q_launch]
    avg_ms = sum(steady) / max(len(steady), 1)
    flops_per_launch = 4.0 * H * D * q_launch * n_local
    achieved = flops_per_launch / (avg_ms * 1e-3) / 1e12 if steady else 0.0
    glob_keys = KNOBS["topk"] * KNOBS["block_size"] + KNOBS["n_init"] + exc
    glob = [ms for r in runs for ms, nq, nk in r[1] if nq == exc and nk == glob_keys]
    waits = [ms for r in runs for ms, nq, nk in r[2] if nq == exc]
    guesses = [sum(x) for x in zip(*(r[3] for r in runs))]
    res = {
        "metric": "InfLLM attn tokens/s @128K ctx (1 layer, Mistral-7B geom); % HBM/MFMA roofline",
        "value": T * args.steps / dt, "unit": "tokens/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup + len(settle_ms),
        "ms_per_step": dt / args.steps * 1e3, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16", "data": "synthetic",
        "config": {"workload": f"{'config 5' if args.favour else 'config 2'}: one InfLLM layer, {T}-token stream, exc 512, H32/Hkv8/D128, "
                               f"n_init128 n_local4096 bs128 topk16 repr_topk4 max_cached{KNOBS['max_cached_block']} lru, GMM keys"
                               + (f", queries favour {args.favour} components per block" if args.favour else ""),
                   "append_chunk": args.chunk},
        "roofline": {"bound": "mfma", "achieved": achieved, "peak": MFMA_BF16_PEAK_TFLOPS, "unit": "TFLOP/s",
                     "frac": achieved / MFMA_BF16_PEAK_TFLOPS,
                     "traffic": counted_traffic("attn_stage__stream32k.hbm_bytes.txt", "local_stage_traffic_bytes"),
                     "kernel": f"attn_stage_kernel<0, false> (local stage, {q_launch} q x {n_local} visible keys x {H} heads per launch)",
                     "avg_launch_ms": avg_ms, "launches_timed": len(steady),
                     "global_stage_avg_ms": sum(glob) / max(len(glob), 1)},
        "cache": cm_stats,
        # the next block's misses are fetched from its candidates, ahead of the selection: how often the candidates
        # were the selection, and how long the main stream still waited for units (the wait itself costs ~6 us)
        "warmup_detail": {"asked": args.warmup, "settling_steps_ms": [round(x, 2) for x in settle_ms]},
        "fetch_ahead": {"guesses": guesses[0], "confirmed": guesses[1], "stream_wait_avg_ms": sum(waits) / max(len(waits), 1)},
    }
    # what the stream as a whole is bound by: the missed units' way from pinned host memory over PCIe (repairs of wrong
    # guesses come on top of the misses counted here)
    unit_bytes = 2 * HKV * KNOBS["block_size"] * D * 2
    moved, staged = runs[-1][5]
    res["host_link"] = {"missed_units_per_step": cm_stats["misses"], "units_from_host_per_step": moved,
                        "units_from_staging_per_step": staged, "bytes_per_step": moved * unit_bytes,
                        "avg_GBps": moved * unit_bytes / (dt / args.steps) / 1e9,
                        "note": "units_from_host counts every 512 KiB unit that crossed PCIe towards the device: the selections' misses, "
                                "candidates a guess fetched in vain and what its repair brought back; units still in a carve staging slot "
                                "are copied on the device.  PCIe 5.0 x16: 64 GB/s raw; 8 DMA engines move 13 units at 54 GB/s on an idle "
                                "GPU; in the stream 7 engines fetch and the 8th takes the carved units to the host"}
    del q, k, v, out, runs
    if not args.no_extra_legs and not args.favour and T == 131072 and args.max_cached_block == 32:
        res.update(extra_legs(args, dev))
    if not args.no_hbm_leg:
        res["roofline_hbm"], scoring = hbm_leg(dev)
        res["kernels_hbm"] = [scoring, call_lists_entry(dev)] + kernels_hbm_leg(dev)
    if args.cpu_tokens > 0:
        res["cpu_baseline"] = cpu_baseline(min(args.cpu_tokens, 16384), min(os.cpu_count() or 1, 16))
    print(json.dumps(res))


if __name__ == "__main__":
    main()
