"""ctypes binding of libjetfire_amd.so (the C ABI declared in include/jetfire_amd.h).

The library is loaded from the package directory; if it is missing this module raises — there is
no CPU fallback for any operator.
"""
from __future__ import annotations

import ctypes as C
import os

_PKG = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_PKG, "libjetfire_amd.so")

P = C.c_void_p
I = C.c_int
L = C.c_int64
F = C.c_float
Z = C.c_size_t

# name -> (restype, argtypes); must list every symbol of include/jetfire_amd.h
SIGNATURES = {
    "jf_last_error": (C.c_char_p, []),
    "jf_version": (C.c_char_p, []),
    "jf_quant_write_sym": (I, [P, L, L, P, L, I, P, L, L, P, L, L, L, I, I, P]),
    "jf_quant_write_int4_sym_kv": (I, [P, L, L, P, L, L, P, L, I, P, L, L, P, L, L, P, L, L, P, L, L, L, I, P]),
    "jf_shadow_write": (I, [P, L, L, P, L, L, P, L, I, P, P, L, L, L, P]),
    "jf_host_buffer_device_pointer": (I, [P, P]),
    "jf_int3_qk_scores": (I, [P, P, P, P, P, I, I, I, I, I, L, I, I, F, P, P]),
    "jf_intn_qk_scores": (I, [I, P, P, P, P, P, P, I, I, I, I, I, L, I, I, F, P, P]),
    "jf_quant_write_int2_asym": (I, [P, L, L, P, L, I, P, L, L, P, L, L, P, L, L, L, I, P]),
    "jf_unpack": (I, [P, L, P, L, P, L, L, I, I, P, L, P]),
    "jf_int8tc_qk_scores": (I, [P, P, P, P, P, I, I, I, I, I, L, I, F, P, P]),
    "jf_topk_slots": (I, [P, P, P, I, I, I, I, I, I, P, P, P, P, P]),
    "jf_softmax_v_workspace_bytes": (Z, [I, I, I]),
    "jf_softmax_v_pre_corr": (I, [P, P, P, P, P, P, P, P, I, I, I, I, I, L, I, I, I, I, P, P, P, P, Z, P]),
    "jf_softmax_v_int8_tiles": (I, [P, P, P, P, P, P, P, P, I, I, I, I, I, L, I, I, P, P, P, P, Z, P]),
    "jf_fused_workspace_bytes": (Z, [I, I, I, I, I, I]),
    "jf_fused_scan_topk": (I, [I, I, P, P, P, P, P, P, P, I, I, I, I, I, L, I, F, I, P, P, P, P, P, P, P, P, P, Z, P]),
    "jf_fused_scan_topk_blend": (I, [I, I, P, P, P, P, P, P, P, I, I, I, I, I, L, I, F, I, P, P, P, P, P, P, P, P, P, P, P, Z, P]),
    "jf_stage_a_topk": (I, [I, I, P, P, P, P, P, I, I, I, I, I, L, I, F, I, P, P, P, P, P, P, Z, P]),
    "jf_stage_a_topk_asym": (I, [I, P, P, P, P, P, P, I, I, I, I, I, L, I, F, I, P, P, P, P, P, P, Z, P]),
    "jf_fused_scan_topk_asym": (I, [I, I, P, P, P, P, P, P, P, P, I, I, I, I, I, L, I, F, I, P, P, P, P, P, P, P, P, P, P, P, Z, P]),
    "jf_topk_slots_fast_workspace_bytes": (Z, [I, I, I, I]),
    "jf_topk_slots_fast": (I, [P, P, P, I, I, I, I, I, I, P, P, P, P, P, Z, P]),
    "jf_stage_b_softmax_v": (I, [I, I, P, P, P, P, P, P, I, I, I, I, I, L, I, I, P, P, P, P, Z, P]),
    "jf_fused_scan_topk_static": (I, [I, I, P, P, P, P, P, P, P, I, I, I, I, I, L, I, F, I, P, P, P, P, P, P, P, P, P]),
    "jf_fused_plan": (I, [I, I, I, I, I, I, I, P, P, P, P]),
    "jf_blend_unnorm": (I, [P, P, P, P, P, I, I, I, P]),
    "jf_cpu_topk_attn": (I, [P, P, P, P, P, P, I, I, I, I, L, F, P]),
    "jf_set_cpu_attn_threads": (I, [I]),
    "jf_get_cpu_attn_threads": (I, []),
    "jf_handoff_create": (P, [I, I, I, I, L, P, P, F]),
    "jf_handoff_submit": (I, [P, P, P, P]),
    "jf_handoff_wait": (I, [P, P, P]),
    "jf_handoff_submit_count": (L, [P]),
    "jf_handoff_stream_submit": (I, [P, P, P, P]),
    "jf_handoff_stream_wait": (I, [P, P, P]),
    "jf_handoff_stream_wait_blend": (I, [P, P, P, P, P, P, P]),
    "jf_handoff_status": (I, [P]),
    "jf_handoff_set_device_wait_limit_us": (I, [P, L]),
    "jf_handoff_set_output_sanitize": (I, [P, I]),
    "jf_handoff_destroy": (None, [P]),
    "jf_blend": (I, [P, P, P, P, P, I, I, I, P]),
    "jf_set_cpu_attn_isa": (I, [I]),
    "jf_get_cpu_attn_isa": (I, []),
    "jf_cpu_topk_sanitize_count": (L, []),
    "jf_submit_ctx_create": (L, [P, P, P, P, P, P, I, I, I, I, L, F, P]),
    "jf_submit_ctx_stream_submit": (I, [L, P]),
    "jf_submit_ctx_stream_wait": (I, [L, P]),
    "jf_submit_ctx_status": (I, [L]),
    "jf_stream_write_value64": (I, [P, P, L]),
    "jf_stream_wait_value64": (I, [P, P, L]),
    "jf_stream_wait_timeouts": (L, []),
    "jf_cpu_topk_attn_async": (I, [P, P, P, P, P, P, I, I, I, I, L, F, P]),
    "jf_wait_for_flag": (I, [P, C.c_double]),
    "jf_graph_pool_warmup": (I, [I]),
    "jf_graph_submit_count": (L, []),
    "jf_reset_graph_runtime_state": (I, []),
    "jf_clear_graph_contexts": (I, []),
    "jf_shadow_append_count": (I, [P, I]),
    "jf_reset_graph_submit_count": (I, []),
    "jf_graph_timing_stats": (I, [P, I]),
    "jf_pool_wake": (I, []),
    "jf_pool_doorbell": (I, [P]),
}

# the measurement / test hooks of include/jetfire_amd_debug.h: present only in a library built with -DJF_DEBUG_HOOKS
DEBUG_SIGNATURES = {
    "jf_calibrate_stream_read": (I, [P, Z, P, P]),
    "jf_profile_scan_begin": (I, [I]),
    "jf_profile_scan_end": (I, [P, P]),
    "jf_debug_phase_clock": (I, [P]),
    "jf_debug_split_len": (I, [I]),
    "jf_debug_pool_stall": (I, [L, I]),
    "jf_debug_pool_wait_stragglers": (I, [I]),
    "jf_handoff_debug_pause": (I, [P, I]),
    "jf_debug_wait_log": (I, [P, I]),
}

_lib = None


def load() -> C.CDLL:
    """Load the shared library (once) and attach the signatures."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise RuntimeError(
            f"{LIB_PATH} is missing: build it with `python -m jetfire_amd.build` "
            "(the HIP library is the only implementation; there is no fallback)")
    lib = C.CDLL(LIB_PATH)
    for name, (res, args) in SIGNATURES.items():
        fn = getattr(lib, name)
        fn.restype = res
        fn.argtypes = args
    for name, (res, args) in DEBUG_SIGNATURES.items():
        fn = getattr(lib, name, None)
        if fn is not None:
            fn.restype = res
            fn.argtypes = args
    _lib = lib
    return lib


def has_debug_hooks() -> bool:
    """Whether the loaded library was built with -DJF_DEBUG_HOOKS (tests and bench.py need that build)."""
    return load().jf_version().decode().endswith("+debug-hooks")


def debug_hook(name: str):
    """A hook of include/jetfire_amd_debug.h, or a RuntimeError that says which build has it."""
    fn = getattr(load(), name, None) if name in DEBUG_SIGNATURES else None
    if fn is None or not has_debug_hooks():
        raise RuntimeError(f"{name} is a measurement / test hook: rebuild with `python -m jetfire_amd.build --debug-hooks`")
    return fn


def check(rc: int) -> None:
    if rc != 0:
        msg = load().jf_last_error().decode("utf-8", "replace")
        raise RuntimeError(msg or f"jetfire_amd call failed with status {rc}")
