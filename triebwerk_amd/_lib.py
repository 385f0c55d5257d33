"""ctypes binding of ``libtriebwerk_kv.so`` (the C ABI in ``include/triebwerk_kv.h``).

The library is the product; there is no Python or CPU fallback.  If the shared
object is missing, loading raises with the command that builds it.
"""
from __future__ import annotations

import ctypes as C
from pathlib import Path

LIB_PATH = Path(__file__).resolve().parent / "lib" / "libtriebwerk_kv.so"

P = C.c_void_p
I = C.c_int
LL = C.c_longlong
SZ = C.c_size_t


class LayerStepArgs(C.Structure):
    """tw_layer_step_args of include/triebwerk_kv.h."""
    _fields_ = [("out", P), ("q", P), ("k", P), ("v", P),
                ("G", I), ("num_heads", I), ("num_kv_heads", I), ("head_dim", I), ("q_dim", I), ("kv_dim", I),
                ("positions", P), ("max_seq_len", I),
                ("q_weight", P), ("k_weight", P), ("eps", C.c_float), ("biased", I),
                ("cos_table", P), ("sin_table", P), ("rope_dim", I),
                ("kv_bits", I), ("cache_k", P), ("cache_v", P), ("k_norms", P), ("v_norms", P), ("rotation", P),
                ("scratch", P), ("gate", P), ("gate_stride", LL), ("ctx_min", I), ("ctx_max", I), ("tickets", P)]


class ModelShape(C.Structure):
    _fields_ = [("num_layers", I), ("num_heads", I), ("num_kv_heads", I), ("head_dim", I)]


# name -> (restype, argtypes).  Order and meaning follow include/triebwerk_kv.h.
SIGNATURES = {
    # Part 1: the reference engine's launchers (engine.cpp:105-171)
    "launch_kv_cache_write_batch": (None, [P, P, P, P, P, I, I, I, P]),
    "launch_turbo_kv_quantize": (None, [P, P, P, P, P, I, I, I, I, I, I, P]),
    "launch_turbo_kv_quantize_batch": (None, [P, P, P, P, P, I, I, I, I, I, I, P]),
    "launch_gqa_attention": (None, [P, P, P, P, P, I, I, I, I, I, P]),
    "launch_gqa_attention_batch": (None, [P, P, P, P, P, P, I, I, I, I, I, I, I, P]),
    "launch_turbo_gqa_attention": (None, [P, P, P, P, P, P, P, P, I, I, I, I, I, I, P]),
    "launch_turbo_gqa_attention_batch": (None, [P, P, P, P, P, P, P, P, P, I, I, I, I, I, I, I, I, P]),
    "launch_gqa_prefill_attention": (None, [P, P, P, P, P, I, I, I, I, I, I, I, P]),
    "launch_turbo_gqa_prefill_attention": (None, [P, P, P, P, P, P, P, P, I, I, I, I, I, I, I, I, P]),
    "launch_increment_positions": (None, [P, I, P]),
    "launch_qk_norm_batch": (None, [P, P, P, P, I, I, I, I, C.c_float, I, I, P, C.c_bool]),
    "launch_rope_batch": (None, [P, P, P, P, P, I, I, I, I, I, I, I, I, P]),
    "launch_qk_norm": (None, [P, P, P, P, I, I, I, C.c_float, P]),
    "launch_rope": (None, [P, P, P, P, I, I, I, I, I, P]),
    "launch_sigmoid_gate_batch": (None, [P, P, I, I, P]),
    # Part 2
    "tw_kv_last_error": (I, []),
    "tw_kv_last_error_string": (C.c_char_p, []),
    "tw_kv_clear_error": (None, []),
    "tw_kv_build_info": (C.c_char_p, []),
    "tw_kv_debug_set_attention_variant": (None, [I]),
    "tw_kv_debug_get_attention_variant": (I, []),
    "tw_kv_debug_set_num_splits": (None, [I]),
    "tw_kv_debug_set_prefill_form": (None, [I]),
    "tw_kv_debug_set_decode_fused": (None, [I]),
    "tw_kv_debug_last_scan_kernel": (C.c_char_p, []),
    "tw_kv_decode_fused_launches": (LL, []),
    "tw_kv_decode_step_plan": (I, [I, I, I, I, I, I, I]),
    "tw_kv_decode_step_plan2": (I, [I, I, I, I, I, I, I, I]),
    "tw_kv_debug_set_fused_shape": (None, [I, I]),
    "tw_kv_debug_profile_attention": (None, [I]),
    "tw_kv_debug_profile_read": (I, [C.POINTER(C.c_double), C.POINTER(I)]),
    "tw_kv_measure_read_bandwidth": (C.c_double, [P, C.c_size_t, I, P]),
    "tw_kv_broadcast_rows": (I, [P, P, P, I, I, I, I, P]),
    "tw_attention_workspace_floats": (SZ, [I, I, I]),
    "tw_turbo_kv_append_batch": (None, [P, P, P, P, P, P, P, P, I, I, I, I, I, I, P]),
    "tw_turbo_kv_append_tokens": (None, [P, P, P, P, P, P, P, P, I, I, I, I, I, I, P]),
    "tw_append_attention_batch": (None, [P, P, P, P, P, P, P, P, I, I, I, I, I, I, I, P]),
    "tw_turbo_append_attention_batch": (None, [P, P, P, P, P, P, P, P, P, P, P, I, I, I, I, I, I, I, I, P]),
    "tw_qk_norm_rope_turbo_append_attention_batch": (None, [P, P, P, P, P, P, C.c_float, I, P, P, I, P, P, P, P, P, P, P,
                                                            I, I, I, I, I, I, I, I, P]),
    "tw_qk_norm_rope_append_attention_batch": (None, [P, P, P, P, P, P, C.c_float, I, P, P, I, P, P, P, P,
                                                      I, I, I, I, I, I, I, P]),
    "tw_layer_attention_step": (None, [C.POINTER(LayerStepArgs), P]),
    "tw_layer_prompt_step": (None, [C.POINTER(LayerStepArgs), P]),
    "tw_paged_kv_cache_write_batch": (None, [P, P, P, P, P, P, I, I, I, P]),
    "tw_paged_turbo_kv_append_batch": (None, [P, P, P, P, P, P, P, P, P, I, I, I, I, I, I, P]),
    "tw_paged_gqa_attention_batch": (None, [P, P, P, P, P, P, P, I, I, I, I, I, I, I, I, P]),
    "tw_paged_turbo_gqa_attention_batch": (None, [P, P, P, P, P, P, P, P, P, P, I, I, I, I, I, I, I, I, I, P]),
    "tw_paged_turbo_append_attention_batch": (None, [P, P, P, P, P, P, P, P, P, P, P, P, I, I, I, I, I, I, I, I, I, P]),
    "tw_turbo_gqa_attention_batch_noalloc": (I, [P, P, P, P, P, P, P, P, I, I, I, I, I, I, I, I, P]),
    "tw_make_rotation_host": (None, [P, I, C.c_uint]),
    # Engine
    "tw_engine_create": (P, [I, I]),
    "tw_engine_destroy": (None, [P]),
    "tw_engine_kv_bits": (I, [P]),
    "tw_engine_max_seq_len": (I, [P]),
    "tw_engine_set_shape": (I, [P, C.POINTER(ModelShape)]),
    "tw_engine_alloc_batch": (I, [P, I, I]),
    "tw_engine_set_arena": (I, [P, P, SZ]),
    "tw_engine_arena_bytes_needed": (SZ, [P, I, I]),
    "tw_engine_reset": (I, [P]),
    "tw_engine_cache_ptr": (P, [P, I, I]),
    "tw_engine_positions": (P, [P]),
    "tw_engine_rotation": (P, [P]),
    "tw_engine_set_positions": (I, [P, P, I]),
    "tw_engine_set_producers": (I, [P, I, P, P, C.c_float, I, P, P, I]),
    "tw_engine_sleep": (I, [P]),
    "tw_engine_wake": (I, [P]),
    "tw_engine_is_allocated": (I, [P]),
    "tw_engine_begin_generation": (I, [P, I, I, P, I]),
    "tw_engine_record_tokens": (I, [P, P, I, P]),
    "tw_engine_check_stops": (I, [P, I, P, C.POINTER(I)]),
    "tw_engine_output": (I, [P, I, C.POINTER(C.POINTER(I)), C.POINTER(I)]),
    "tw_engine_host_position": (I, [P, I]),
    "tw_engine_layer_step": (I, [P, I, P, P, P, P, P]),
    "tw_engine_prompt_layer": (I, [P, I, I, P, P, P, P, P, I, P]),
    "tw_engine_decode_step": (I, [P, P, P, P, P, I, P]),
    "tw_engine_broadcast_prefix": (I, [P, I, I, I, I, P]),
    "tw_engine_graph_state": (I, [P]),
    "tw_engine_debug_fail_captures": (None, [P, I]),
    "tw_kv_set_trace_ranges": (I, [I]),
    "tw_engine_alloc_single": (I, [P]),
    "tw_engine_single_is_allocated": (I, [P]),
    "tw_engine_single_cache_ptr": (P, [P, I, I]),
    "tw_engine_single_rotation": (P, [P]),
    "tw_engine_single_pos": (I, [P]),
    "tw_engine_single_set_pos": (I, [P, I]),
    "tw_engine_single_step": (I, [P, I, P, P, P, P, P]),
    "tw_engine_single_advance": (I, [P, P]),
}

_lib = None


class LibraryMissing(RuntimeError):
    pass


def load() -> C.CDLL:
    """Load the shared library once and attach the signatures."""
    global _lib
    if _lib is not None:
        return _lib
    if not LIB_PATH.exists():
        raise LibraryMissing(
            f"{LIB_PATH} is not built. Build it with `python -m triebwerk_amd.build` "
            "(needs hipcc); there is no fallback path."
        )
    lib = C.CDLL(str(LIB_PATH))
    for name, (restype, argtypes) in SIGNATURES.items():
        fn = getattr(lib, name)  # AttributeError here = header and library disagree
        fn.restype = restype
        fn.argtypes = argtypes
    _lib = lib
    return lib


def check(lib: C.CDLL | None = None) -> None:
    """Raise if a launcher recorded an error since the last clear."""
    lib = lib or load()
    code = lib.tw_kv_last_error()
    if code != 0:
        msg = lib.tw_kv_last_error_string().decode()
        lib.tw_kv_clear_error()
        raise RuntimeError(f"triebwerk_kv error {code}: {msg}")
