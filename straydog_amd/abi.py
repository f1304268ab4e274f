"""ctypes declarations of the C ABI in include/straydog_gpu.h and include/straydog_gpu_ext.h.

This is the Python counterpart of the reference's generated Rust bindings (crates/straydog-gpu/src/ffi.rs):
one declaration per exported function, nothing else.  Loading fails loudly when the HIP library has not
been built; there is no CPU fallback.
"""
import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIBRARY = os.path.join(_HERE, "libstraydog_gpu.so")

c_void_p, c_int, c_u64, c_u32, c_i64, c_float, c_size_t = (
    ctypes.c_void_p, ctypes.c_int, ctypes.c_uint64, ctypes.c_uint32, ctypes.c_int64, ctypes.c_float, ctypes.c_size_t)


class KvPool(ctypes.Structure):
    """sdx_kv_pool"""
    _fields_ = [("pages", c_void_p), ("page_count", c_u64), ("page_tokens", c_u32), ("kv_heads", c_u32), ("dim", c_u32),
                ("row_bytes", c_u32)]


_P = ctypes.POINTER


class QsaState(ctypes.Structure):
    """sdx_qsa_state"""
    _fields_ = [("kv", _P(KvPool)), ("page_table", c_void_p), ("context", c_u64), ("blocks", c_void_p), ("history", c_void_p), ("q_norm", c_void_p),
                ("k_norm", c_void_p), ("index_q_norm", c_void_p), ("index_k_norm", c_void_p), ("heads", c_u64)]

# name -> (restype, argtypes); the order is that of the headers
SIGNATURES = {
    # straydog_gpu.h
    "sd_error": (ctypes.c_char_p, []),
    "sd_device_count": (c_int, []),
    "sd_device_info": (c_int, [c_int, ctypes.c_char_p, c_size_t, _P(c_u64), _P(c_u64)]),
    "sd_create": (c_void_p, [c_int, c_u64]),
    "sd_destroy": (None, [c_void_p]),
    "sd_memory": (c_int, [c_void_p, _P(c_u64), _P(c_u64)]),
    "sd_upload": (c_void_p, [c_void_p, c_void_p, c_u64]),
    "sd_allocate": (c_void_p, [c_void_p, c_u64]),
    "sd_write": (c_int, [c_void_p, c_void_p, c_void_p, c_u64]),
    "sd_release": (c_int, [c_void_p, c_void_p]),
    "sd_allocation_bytes": (c_int, [c_void_p, c_void_p, _P(c_u64)]),
    "sd_zero": (c_int, [c_void_p, c_void_p]),
    "sd_download": (c_int, [c_void_p, c_void_p, c_void_p, c_u64]),
    "sd_buffer": (c_void_p, [c_void_p, c_u64]),
    "sd_buffer_write": (c_int, [c_void_p, c_void_p, c_u64, c_void_p, c_u64]),
    "sd_buffer_read": (c_int, [c_void_p, c_void_p, c_u64, c_void_p, c_u64]),
    "sd_graph_begin": (c_int, [c_void_p]),
    "sd_graph_end": (c_int, [c_void_p, c_u64, c_int]),
    "sd_graph_run": (c_int, [c_void_p, c_u64]),
    "sd_checkpoint_buffer": (c_void_p, [c_void_p, c_u64]),
    "sd_checkpoint_copy": (c_int, [c_void_p, c_int, _P(c_void_p), c_u64, c_void_p]),
    "sd_checkpoint_clone": (c_int, [c_void_p, c_void_p, c_void_p]),
    "sd_state_copy": (c_int, [c_void_p, c_void_p, c_u64, c_u64, c_u64, c_u64, c_void_p, c_u64, c_int]),
    "sdx_checkpoint_release": (c_int, [c_void_p, c_void_p]),
    "sd_kv_format": (c_int, [c_void_p, c_u32]),
    "sd_kv_stage": (c_int, [c_void_p, c_void_p, c_u64]),
    "sd_host_state": (c_void_p, [c_void_p, c_u64]),
    "sd_host_state_supported": (c_int, [c_void_p]),
    "sd_host_states_prefetch": (c_int, [c_void_p, _P(c_u64), c_u64]),
    "sd_attention_sequence": (c_int, [c_void_p, c_void_p, c_u64, c_u64, c_u64, c_u64, c_void_p, c_u64, c_void_p, c_u64]),
    "sd_op_attention": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_u64, c_void_p, c_u64, c_u64, c_u64, c_u64, c_float,
                                c_void_p, c_void_p, c_u64, c_void_p]),
    "sd_op_sparse_attention": (c_int, [c_void_p, c_void_p, c_void_p, c_u64, c_void_p, c_u64, c_void_p, c_u64, c_void_p, c_u64,
                                       c_void_p, c_u64, c_u64, c_u64, c_float, c_u64, c_void_p, c_void_p, c_u64, c_void_p]),
    "sd_op_rope": (c_int, [c_void_p, c_void_p, c_u64, c_u64, c_u64, c_u64, c_void_p, c_void_p, c_int]),
    "sd_op_compress": (c_int, [c_void_p, c_void_p, c_void_p, c_u64, c_u64, c_u64, c_void_p]),
    "sd_op_index_scores": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_u64, c_u64, c_u64, c_u64, c_float, c_void_p]),
    "sd_op_top_k": (c_int, [c_void_p, c_void_p, c_u64, c_u64, c_u64, c_void_p]),
    "sd_op_index_candidates": (c_int, [c_void_p, c_void_p, c_void_p, c_u64, c_u64, c_u64, c_u64, c_void_p, c_void_p, c_u64]),
    "sd_op_index_select": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_u64, c_u64, c_u64, c_u64, c_float, c_u64,
                                   c_void_p, c_void_p, c_void_p, c_u64, c_void_p, c_void_p, c_u64, c_u64]),
    "sd_op_index_select_proj": (c_int, [c_void_p, c_void_p, c_int, c_u64, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_u64, c_u64, c_u64,
                                        c_float, c_u64, c_void_p, c_void_p, c_void_p, c_u64, c_void_p, c_void_p, c_u64, c_u64]),
    "sd_op_to_bf16": (c_int, [c_void_p, c_void_p, c_u64, c_void_p]),
    # straydog_gpu_ext.h
    "sd_op_dspark_attention": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_u64, c_u64, ctypes.c_uint32, c_void_p, c_u64, c_void_p]),
    "sd_op_split": (c_int, [c_void_p, c_void_p, c_u64, c_u64, c_void_p, c_void_p]),
    "sd_op_rms_norm": (c_int, [c_void_p, c_void_p, c_void_p, c_u64, c_u64, c_float, c_void_p]),
    "sd_op_norm_rope": (c_int, [c_void_p, c_void_p, c_void_p, c_u64, c_u64, c_float, c_u64, c_void_p, c_void_p, c_void_p, c_void_p, c_u64]),
    "sd_attention_turns_reserve": (c_int, [c_void_p, c_u64, c_u64]),
    "sd_attention_turns_arm": (c_int, [c_void_p, c_u64]),
    "sd_op_rope_halves": (c_int, [c_void_p, c_void_p, c_u64, c_u64, c_u64, c_u64, c_void_p, c_void_p]),
    "sd_op_scatter": (c_int, [c_void_p, c_void_p, c_void_p, c_u64, c_u64, c_void_p, c_u64]),
    "sd_op_attention_prepare": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_u64, c_u64, c_u64, c_u64, c_void_p, c_void_p, c_float, c_u64,
                                        c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_u64]),
    "sdx_kv_cache_create": (c_void_p, [c_void_p, c_u64, ctypes.c_uint32, ctypes.c_uint32, ctypes.c_uint32, ctypes.c_uint32, c_u64, c_u64]),
    "sdx_kv_cache_destroy": (c_int, [c_void_p, c_void_p]),
    "sdx_kv_cache_view": (c_int, [c_void_p, c_void_p, _P(KvPool), _P(c_void_p), _P(c_u64)]),
    "sdx_kv_cache_reserve": (c_int, [c_void_p, c_void_p, c_u64, c_u64]),
    "sdx_kv_cache_truncate": (c_int, [c_void_p, c_void_p, c_u64, c_u64]),
    "sdx_kv_cache_fork": (c_int, [c_void_p, c_void_p, c_u64, c_u64, c_u64]),
    "sdx_kv_cache_usage": (c_int, [c_void_p, c_void_p, c_u64, _P(c_u64), _P(c_u64)]),
    "sdx_kv_cache_host": (c_int, [c_void_p, c_void_p, c_u64]),
    "sdx_kv_cache_park": (c_int, [c_void_p, c_void_p, c_u64]),
    "sdx_kv_cache_resume": (c_int, [c_void_p, c_void_p, c_u64]),
    "sdx_kv_cache_stage": (c_int, [c_void_p, c_void_p, c_u64, c_u64, _P(KvPool), _P(c_void_p), _P(c_u64)]),
    "sdx_kv_cache_unstage": (c_int, [c_void_p, c_void_p, c_u64, c_u64, c_u64]),
    "sdx_kv_cache_grow": (c_int, [c_void_p, c_void_p, c_u64]),
    "sdx_kv_cache_residency": (c_int, [c_void_p, c_void_p, c_u64, _P(c_u64), _P(c_u64), _P(c_u64)]),
    "sdx_kv_cache_gather": (c_int, [c_void_p, c_void_p, c_u64, c_u64, c_u64, c_void_p, c_u64, c_void_p, c_u64, c_u64, c_void_p, _P(c_u64), _P(c_u64), _P(KvPool),
                                    _P(c_void_p), _P(c_u64)]),
    "sdx_kv_write": (c_int, [c_void_p, _P(KvPool), c_void_p, c_u64, c_void_p, c_void_p, c_void_p, c_int, c_u64, c_u64]),
    "sdx_paged_attention_scratch": (c_u64, [c_u64, c_u64, c_u64, c_u64, c_u64]),
    "sdx_paged_attention": (c_int, [c_void_p, _P(KvPool), c_void_p, c_u64, c_void_p, c_u64, c_void_p, c_int, c_u64, c_u64, c_u64,
                                    c_float, c_void_p, c_int, c_void_p, c_u64]),
    "sdx_prefill_tiles_bytes": (c_u64, [c_u64, c_u64, c_u64, c_u64]),
    "sdx_prefill_wave_rows": (c_int, [c_void_p, c_u64]),
    "sdx_prefill_chunk": (c_int, [c_void_p, _P(KvPool), c_void_p, c_u64, c_void_p, c_u64, c_void_p, c_void_p, c_int, c_void_p, c_int, c_u64, c_u64,
                                  c_u64, c_float, c_void_p, c_int, c_void_p, c_u64, c_void_p]),
    "sdx_paged_attention_static_bytes": (c_u64, []),
    "sdx_paged_attention_static": (c_int, [c_void_p, _P(KvPool), c_void_p, c_u64, c_void_p, c_u64, c_void_p, c_int, c_u64, c_u64, c_u64,
                                           c_float, c_void_p, c_int]),
    "sdx_qsa_normalize": (c_int, [c_void_p, c_void_p, c_void_p, c_u64, c_u64, c_u64, c_u64, c_u64, c_void_p]),
    "sdx_qsa_pool": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_u64, c_u64, c_u64, c_void_p]),
    "sdx_qsa_index_interval_scratch": (c_u64, [c_u64, c_u64]),
    "sdx_qsa_index_interval": (c_int, [c_void_p, c_void_p, c_u64, c_void_p, c_u64, c_u64, c_u64, c_u64, c_void_p, c_void_p, c_void_p, c_void_p, c_u64,
                                       _P(c_u64)]),
    "sdx_qsa_index_interval_undecided": (c_int, [c_void_p, c_void_p, c_u64, c_u64, _P(c_u64)]),
    "sdx_qsa_index": (c_int, [c_void_p, c_void_p, c_u64, c_void_p, c_u64, c_u64, c_void_p, c_u64, c_u64, c_void_p, c_void_p, c_void_p]),
    "sdx_selected_attention_scratch": (c_u64, [c_u64, c_u64, c_u64]),
    "sdx_selected_attention": (c_int, [c_void_p, _P(KvPool), c_void_p, c_u64, c_u64, c_void_p, c_void_p, c_u64, c_void_p, c_void_p, c_int,
                                       c_u64, c_u64, c_float, c_void_p, c_u64, c_u64, c_void_p, c_int, c_void_p, c_u64]),
    "sdx_selected_attention_union_scratch": (c_u64, [c_u64, c_u64, c_u64, c_u64, c_u64]),
    "sdx_selected_attention_union": (c_int, [c_void_p, _P(KvPool), c_void_p, c_u64, c_u64, c_void_p, c_u64, c_void_p, c_void_p, c_int,
                                             c_u64, c_u64, c_float, c_void_p, c_u64, c_u64, c_void_p, c_int, c_void_p, c_u64]),
    "sdx_qsa_decode_attend_scratch": (c_u64, [c_u64, c_u64, c_u64, c_u64]),
    "sdx_qsa_decode_attend": (c_int, [c_void_p, _P(QsaState), c_void_p, c_u64, c_u64, c_void_p, c_void_p, c_void_p, c_u64, c_void_p]),
    "sdx_qsa_prefill_attend_scratch": (c_u64, [c_u64, c_u64, c_u64, c_u64]),
    "sdx_qsa_prefill_attend": (c_int, [c_void_p, _P(QsaState), c_void_p, c_u64, c_u64, c_u64, c_void_p, c_u64, _P(c_u64), c_void_p]),
    "sdx_index_projection": (c_int, [c_void_p, c_void_p, c_int, c_u64, c_void_p, c_u64, c_void_p]),
    "sdx_index_score_bounds": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_u64, c_u64, c_u64, c_u64, c_float, c_void_p, c_void_p]),
    "sdx_index_top_k": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_u64, c_u64, c_u64, c_u64, c_float, c_void_p,
                                c_u64, c_void_p]),
    "sdx_latent_attention": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_u64, c_u64, c_u64, c_u64, c_u64, c_u64, c_float,
                                     c_void_p]),
    "sdx_synchronize": (c_int, [c_void_p]),
    "sdx_event_record": (c_i64, [c_void_p]),
    "sdx_event_elapsed": (c_int, [c_void_p, c_i64, c_i64, _P(c_float)]),
    "sdx_events_clear": (c_int, [c_void_p]),
    "sdx_device_compute_units": (c_int, [c_void_p]),
    "sdx_device_state": (c_int, [c_void_p, c_void_p]),
    "sdx_profile": (c_int, [c_void_p, c_int]),
    "sdx_profile_read": (c_int, [c_void_p, _P(ctypes.c_double), _P(c_u64)]),
    "sdx_fill_normal": (c_int, [c_void_p, c_void_p, c_u64, c_u64, c_int]),
    "sdx_fill_uniform": (c_int, [c_void_p, c_void_p, c_u64, c_u64, c_float, c_float]),
    "sdx_copy": (c_int, [c_void_p, c_void_p, c_void_p, c_u64]),
    "sdx_read_probe": (c_int, [c_void_p, c_void_p, c_u64, c_u32, c_u32]),
    "sdx_paged_stream_probe": (c_int, [c_void_p, _P(KvPool), _P(c_u64)]),
    "sdx_mfma_probe": (c_int, [c_void_p, c_u32, c_int, _P(ctypes.c_double)]),
}


def load(path=LIBRARY):
    """The library with every function of the two headers typed; raises if it is missing or lacks a symbol."""
    if not os.path.exists(path):
        raise RuntimeError(f"{path} is not built: run `python -m straydog_amd.build` (hipcc, gfx950); there is no CPU fallback")
    library = ctypes.CDLL(path)
    for name, (restype, argtypes) in SIGNATURES.items():
        function = getattr(library, name)     # AttributeError names the missing symbol
        function.restype = restype
        function.argtypes = argtypes
    return library
