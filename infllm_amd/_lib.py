"""ctypes binding of libinfllm_hip.so (the C ABI declared in include/infllm_hip.h).

The library is the only compute path of this package: if it is missing or does
not export the expected symbols, loading raises - there is no fallback.
"""
import ctypes as C
import os

LIB_PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "libinfllm_hip.so")
ABI_VERSION = 1

c_i32, c_i64, c_f32, c_f64, c_vp = C.c_int32, C.c_int64, C.c_float, C.c_double, C.c_void_p


class IngestArgs(C.Structure):
    _fields_ = [
        ("d_q", c_vp), ("d_k", c_vp), ("d_v", c_vp),
        ("q_sb", c_i64), ("q_sh", c_i64), ("q_sl", c_i64),
        ("k_sb", c_i64), ("k_sh", c_i64), ("k_sl", c_i64),
        ("v_sb", c_i64), ("v_sh", c_i64), ("v_sl", c_i64),
        ("B", c_i32), ("H", c_i32), ("Hkv", c_i32), ("n", c_i32),
        ("pos0", c_i64), ("glb_pos", c_i64),
        ("d_inv_freq", c_vp), ("distance_scale", c_f64),
        ("d_ring_k_raw", c_vp), ("d_ring_k_rot", c_vp), ("d_ring_v", c_vp),
        ("d_ring_score", c_vp), ("ring_cap", c_i64),
        ("d_q_loc", c_vp), ("d_q_glb", c_vp), ("d_qpart", c_vp),
    ]


class Page(C.Structure):
    _fields_ = [("k", c_vp), ("v", c_vp), ("head_stride", c_i64), ("n_valid", c_i32), ("reserved", c_i32)]


class AttnArgs(C.Structure):
    _fields_ = [
        ("d_q", c_vp), ("q_sb", c_i64), ("q_sh", c_i64), ("q_sl", c_i64),
        ("B", c_i32), ("H", c_i32), ("Hkv", c_i32), ("Lq", c_i32),
        ("d_k", c_vp), ("d_v", c_vp),
        ("k_sb", c_i64), ("k_sh", c_i64), ("k_sl", c_i64),
        ("v_sb", c_i64), ("v_sh", c_i64), ("v_sl", c_i64),
        ("cap", c_i64), ("j_lo", c_i64), ("j_hi", c_i64),
        ("mask", c_i32), ("reserved", c_i32),
        ("offset", c_i64), ("window", c_i64),
        ("d_pages", c_vp), ("n_pages", c_i32), ("nsplit", c_i32),
        ("softmax_scale", c_f32),
        ("d_o_part", c_vp), ("d_lse_part", c_vp),
    ]


class ScoreArgs(C.Structure):
    _fields_ = [
        ("d_q", c_vp), ("q_sb", c_i64), ("q_sh", c_i64), ("q_sl", c_i64),
        ("B", c_i32), ("H", c_i32), ("Hkv", c_i32), ("Lq", c_i32),
        ("d_k", c_vp), ("k_sb", c_i64), ("k_sh", c_i64), ("k_sl", c_i64),
        ("cap", c_i64), ("j_lo", c_i64), ("j_hi", c_i64),
        ("mask", c_i32), ("accumulate", c_i32),
        ("offset", c_i64), ("window", c_i64),
        ("d_lse", c_vp), ("softmax_scale", c_f32), ("n_parts", c_i32),
        ("d_score", c_vp), ("score_sb", c_i64), ("score_sh", c_i64), ("score_cap", c_i64),
    ]


class LayerDesc(C.Structure):
    _fields_ = [
        ("B", c_i32), ("H", c_i32), ("Hkv", c_i32),
        ("n_local", c_i32), ("n_init", c_i32), ("block_size", c_i32), ("exc", c_i32), ("topk", c_i32),
        ("repr_topk", c_i32), ("max_cached", c_i32), ("max_splits", c_i32), ("num_cus", c_i32),
        ("ring_cap", c_i64),
        ("d_ring_k_raw", c_vp), ("d_ring_k_rot", c_vp), ("d_ring_v", c_vp), ("d_ring_score", c_vp),
        ("d_init_kv", c_vp), ("init_cap", c_i64), ("d_slab", c_vp),
        ("d_q_loc", c_vp), ("d_q_glb", c_vp), ("d_qbar", c_vp), ("d_qpart", c_vp),
        ("d_o_part", c_vp), ("d_lse_part", c_vp), ("d_lse", c_vp),
        ("d_topk_idx", c_vp), ("h_topk_idx", c_vp),
        ("d_pages", c_vp), ("h_pages", c_vp), ("max_pages", c_i32), ("page_slots", c_i32),
        ("d_carve_stage", c_vp), ("max_carve", c_i32), ("carve_slots", c_i32),
        ("d_inv_freq", c_vp), ("distance_scale", c_f64), ("softmax_scale", c_f32), ("reserved", c_i32),
        ("d_topk_flag", c_vp), ("h_topk_flag", c_vp),
    ]


class FrontArgs(C.Structure):
    _fields_ = [
        ("d_q", c_vp), ("d_k", c_vp), ("d_v", c_vp),
        ("q_sb", c_i64), ("q_sh", c_i64), ("q_sl", c_i64),
        ("k_sb", c_i64), ("k_sh", c_i64), ("k_sl", c_i64),
        ("v_sb", c_i64), ("v_sh", c_i64), ("v_sl", c_i64),
        ("n", c_i32), ("n_units", c_i32), ("b0", c_i64),
        ("d_reps", c_vp), ("rep_sb", c_i64), ("rep_su", c_i64),
        ("d_unit_scores", c_vp), ("unit_scores_sb", c_i64),
        ("d_q_next", c_vp), ("d_k_next", c_vp), ("d_v_next", c_vp), ("n_next", c_i32), ("flags", c_i32),
        ("d_call_scores", c_vp), ("call_scores_cols", c_i64),
    ]


class BatchDesc(C.Structure):
    _fields_ = [
        ("d_q_loc", c_vp), ("d_q_glb", c_vp), ("d_qpart", c_vp), ("d_qbar", c_vp),
        ("d_o_part", c_vp), ("d_lse_part", c_vp), ("part_rows", c_i64),
        ("max_tokens", c_i32), ("group_blocks", c_i32),
    ]


class BackArgs(C.Structure):
    _fields_ = [
        ("n", c_i32), ("n_sel", c_i32), ("b0", c_i64),
        ("h_sel_slots", c_vp), ("n_miss", c_i32), ("init_len", c_i32),
        ("h_miss_row", c_vp), ("h_miss_slot", c_vp), ("h_miss_unit", c_vp), ("h_miss_src", c_vp),
        ("cursor", c_i64),
        ("d_out", c_vp), ("o_sb", c_i64), ("o_sh", c_i64), ("o_sl", c_i64),
        ("init_take", c_i32), ("n_carve", c_i32),
        ("d_rep_out", c_vp), ("rep_sb", c_i64), ("rep_su", c_i64),
        ("d_repr_idx", c_vp), ("h_carve_dst", c_vp),
        ("n_units", c_i32), ("flags", c_i32), ("d_reps", c_vp), ("d_unit_scores", c_vp), ("unit_scores_sb", c_i64),
        ("d_unit_mass", c_vp), ("d_mass_scratch", c_vp),
    ]


class SelectArgs(C.Structure):
    _fields_ = [
        ("caches", c_vp), ("h_selected", c_vp), ("n_sel", c_i32), ("wait_topk", c_i32),
        ("h_chunk_base", c_vp), ("n_chunks", c_i32), ("units_per_chunk", c_i32),
        ("unit_bytes", c_i64), ("row_bytes", c_i64),
        ("h_sel_slots", c_vp), ("h_miss_row", c_vp), ("h_miss_slot", c_vp), ("h_miss_unit", c_vp), ("h_miss_src", c_vp),
        ("h_evicted", c_vp), ("h_n_evicted", c_vp), ("h_n_miss", c_vp),
    ]


NO_RETRIEVAL = 1            # INFLLM_NO_RETRIEVAL
CACHE_STRATEGY = {"lru": 0, "fifo": 1, "lru-s": 2}      # INFLLM_CACHE_*

# name -> (restype, argtypes); every symbol include/infllm_hip.h declares
SYMBOLS = {
    "infllm_version": (c_i32, []),
    "infllm_last_error": (C.c_char_p, []),
    "infllm_ingest": (c_i32, [C.POINTER(IngestArgs), c_vp]),
    "infllm_reduce_partials": (c_i32, [c_vp, c_i32, c_i32, c_i32, c_f32, c_vp, c_vp]),
    "infllm_block_mean": (c_i32, [c_vp, c_i32, c_i32, c_i32, c_i32, c_vp, c_vp]),
    "infllm_chunk_qbar": (c_i32, [c_vp, c_i64, c_i64, c_i64, c_i32, c_i32, c_i32, c_i32, c_vp, C.c_double, c_i64, c_vp, c_vp]),
    "infllm_rope_rows": (c_i32, [c_vp, c_i64, c_i64, c_i64, c_i32, c_i32, c_i32, c_i64, c_i32, c_vp, C.c_double, c_vp, c_vp]),
    "infllm_attn_stage": (c_i32, [C.POINTER(AttnArgs), c_vp]),
    "infllm_attn_merge": (c_i32, [c_vp, c_vp, c_i32, c_i32, c_i32, c_i32, c_vp, c_i64, c_i64, c_i64, c_vp, c_vp]),
    "infllm_attn_fwd": (c_i32, [C.POINTER(AttnArgs), C.POINTER(AttnArgs), c_vp, c_i64, c_i64, c_i64, c_vp, c_vp]),
    "infllm_attn_stages_fused": (c_i32, [C.POINTER(AttnArgs), C.POINTER(AttnArgs), c_vp]),
    "infllm_attn_fwd_noalloc": (c_i32, [C.POINTER(AttnArgs), C.POINTER(AttnArgs), c_vp, c_i64, c_i64, c_i64, c_vp, c_vp]),
    "infllm_local_score": (c_i32, [C.POINTER(ScoreArgs), c_vp]),
    "infllm_unit_scores": (c_i32, [c_vp, c_i64, c_i32, c_i32, c_i32, c_vp, c_vp, c_vp]),
    "infllm_topk": (c_i32, [c_vp, c_i32, c_i32, c_vp, c_vp]),
    "infllm_score_topk": (c_i32, [c_vp, c_i64, c_i32, c_i32, c_vp, c_i32, c_vp, c_vp, c_vp]),
    "infllm_score_topk_queries": (c_i32, [c_vp, c_i64, c_i32, c_i32, c_vp, c_i64, c_i32, c_i32, c_vp, c_i64, c_vp, c_i64, c_vp]),
    "infllm_score_new_topk": (c_i32, [c_vp, c_i64, c_i32, c_vp, c_vp, c_vp, c_i32, c_i32, c_i32, c_i32, c_vp, c_vp]),
    "infllm_repr_keys": (c_i32, [c_vp, c_vp, c_i64, c_i32, c_i32, c_i32, c_i64, c_i32, c_i32, c_i32,
                                 c_vp, c_i64, c_i64, c_vp, c_vp]),
    "infllm_gather_rows": (c_i32, [c_vp, c_i64, c_i32, c_i32, c_i64, c_i32, c_i32, c_vp, c_i64, c_i64, c_i64, c_vp]),
    "infllm_copy_async": (c_i32, [c_vp, c_vp, c_i64, c_i32, c_vp]),
    "infllm_cache_copy_async": (c_i32, [c_vp, c_vp, c_i64, c_i32, c_vp]),
    "infllm_fetch_units": (c_i32, [c_vp, c_vp, c_i32, c_i64, c_vp]),
    "infllm_host_device_pointer": (c_vp, [c_vp]),
    "infllm_layer_create": (c_vp, [C.POINTER(LayerDesc)]),
    "infllm_layer_destroy": (c_i32, [c_vp]),
    "infllm_block_front": (c_i32, [c_vp, C.POINTER(FrontArgs), c_vp]),
    "infllm_layer_set_batch": (c_i32, [c_vp, C.POINTER(BatchDesc)]),
    "infllm_layer_staged_units": (c_i64, [c_vp]),
    "infllm_layer_fetched_units": (c_i64, [c_vp]),
    "infllm_layer_path_counts": (c_i32, [c_vp, c_vp]),
    "infllm_call_front": (c_i32, [c_vp, C.POINTER(FrontArgs), c_vp]),
    "infllm_layer_wait_topk": (c_i32, [c_vp]),
    "infllm_layer_wait_mass": (c_i32, [c_vp]),
    "infllm_block_fetch": (c_i32, [c_vp, c_i32, c_vp, c_vp, c_vp, c_vp, c_vp, c_vp]),
    "infllm_block_back": (c_i32, [c_vp, C.POINTER(BackArgs), c_vp, c_vp]),
    "infllm_layer_flush": (c_i32, [c_vp, c_vp]),
    "infllm_layer_end_call": (c_i32, [c_vp, c_vp]),
    "infllm_cache_create": (c_vp, [c_i32, c_i32, c_f64]),
    "infllm_cache_destroy": (c_i32, [c_vp]),
    "infllm_cache_touch": (c_i32, [c_vp, c_vp, c_i32, c_vp, c_vp, c_vp, c_vp, c_vp]),
    "infllm_cache_touch_hinted": (c_i32, [c_vp, c_vp, c_i32, c_vp, c_vp, c_vp, c_vp, c_vp, c_vp, c_vp, c_i32]),
    "infllm_cache_add_scores": (c_i32, [c_vp, c_vp, c_vp, c_i32]),
    "infllm_cache_residents": (c_i32, [c_vp, c_vp, c_vp, c_vp, c_i32]),
    "infllm_cache_slot_of": (c_i32, [c_vp, c_i32]),
    "infllm_cache_clone": (c_vp, [c_vp]),
    "infllm_cache_copy": (c_i32, [c_vp, c_vp]),
    "infllm_block_select": (c_i32, [c_vp, C.POINTER(SelectArgs), c_vp, c_vp]),
    "infllm_block_prefetch": (c_i32, [c_vp, C.POINTER(SelectArgs), c_vp, c_vp]),
    "infllm_layer_prefetch_stats": (c_i32, [c_vp, c_vp, c_vp]),
    "infllm_layer_last_selection": (c_i32, [c_vp, c_vp, c_i32]),
    "infllm_layer_timing": (c_i32, [c_vp, c_i32, c_i32]),
    "infllm_layer_read_timing": (c_i32, [c_vp, c_i32, c_vp, c_vp, c_vp, c_i32]),
}

_lib = None


class InfLLMHipError(RuntimeError):
    pass


def load():
    """Load the shared library once; raise if it is absent or incomplete."""
    global _lib
    if _lib is not None:
        return _lib
    # One HIP runtime (and one ROCr) per process: PyTorch bundles its own and every device pointer handed to the library
    # comes from it, so it has to be the copy that is loaded first; the library's dependencies then resolve to it.
    import torch  # noqa: F401
    if not os.path.exists(LIB_PATH):
        raise InfLLMHipError(
            f"{LIB_PATH} is missing: build it with `python -m infllm_amd.build` "
            "(hipcc --offload-arch=gfx950); this package has no other compute path")
    lib = C.CDLL(LIB_PATH)
    for name, (restype, argtypes) in SYMBOLS.items():
        try:
            fn = getattr(lib, name)
        except AttributeError as e:
            raise InfLLMHipError(f"{LIB_PATH} does not export {name}") from e
        fn.restype, fn.argtypes = restype, argtypes
    if lib.infllm_version() != ABI_VERSION:
        raise InfLLMHipError(f"ABI version {lib.infllm_version()} != expected {ABI_VERSION}; rebuild the library")
    _lib = lib
    return lib


def check(status, what):
    if status != 0:
        msg = load().infllm_last_error()
        raise InfLLMHipError(f"{what} failed ({status}): {msg.decode() if msg else ''}")
