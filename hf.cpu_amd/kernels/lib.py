"""Loading the kernel library and declaring its C interface (csrc/api.h) to ctypes.

There is no fallback: if the library is missing it is built, and if it cannot be
built or loaded the error is raised to the caller.
"""
import ctypes
import threading
from ctypes import c_char_p, c_float, c_int, c_size_t, c_void_p

from . import build as _build

_lock = threading.Lock()
_lib = None

P, I, F = c_void_p, c_int, c_float
_SIGNATURES = {
    "hfa_embed": [P, I, P, P, I, I, I, P],
    "hfa_rmsnorm": [P, P, P, I, P, I, I, F, P, I, P, P],
    "hfa_gemm": [P, I, I, P, I, I, P, P, I, I, I, I, I, I, I, P, c_size_t, I, P, I, P],
    "hfa_gemm_finish": [P, I, P, P, I, I, I, I, I, I, P],
    "hfa_gemm_rows": [I, P, I, P, I, I, I, I, P, P, I, F, F, P, I, I, I, P, I, P, P, P, I, P, I, P],
    "hfa_gemm_rows_supports": [I, I, I, I, I, I],
    "hfa_rope_store": [P, I, I, P, P, I, I, I, I, I, P, P, P, I, I, P, I, P, P],
    "hfa_paged_attention": [P, I, I, P, P, I, I, P, I, P, P, P, I, I, I, P, I, I, I, I, I, I, I, I, I, F, P, I, I, F, I, P, P, c_size_t, I, P],
    "hfa_scale_add": [P, I, P, F, P, I, I, I, I, P],
    "hfa_gate_mul": [P, I, I, P, I, I, P, I, I, I, I, I, P],
    "hfa_latent_pack": [P, I, P, I, I, P, F, P, I, I, I, I, I, I, I, P, I, P],
    "hfa_channel_scan": [P, I, P, I, P, I, I, P, I, I, I, I, I, I, F, P, c_size_t, P, P, I, P, I, P],
    "hfa_channel_decay": [P, I, I, P, I, P, F, P, I, I, I, P],
    "hfa_group_rmsnorm": [P, I, I, P, P, I, I, P, I, I, I, F, P, I, I, I, P, P],
    "hfa_delta_scan": [P, I, P, I, I, I, P, I, I, I, P, I, P, P, P, I, F, F, P, c_size_t, P, P, I, I, P, I, P],
    "hfa_embed_pos": [P, I, P, P, P, P, I, I, I, F, P],
    "hfa_rmsnorm_add": [P, I, P, I, I, P, P, P, I, I, I, F, F, I, P],
    "hfa_polynorm": [P, I, I, P, P, I, I, I, I, F, P],
    "hfa_scale_rows": [P, I, I, I, F, P],
    "hfa_head_norm_store": [P, I, I, I, I, I, I, P, P, F, P, I, P, P, I, P, I, I, P],
    "hfa_talk_mix": [P, I, P, P, I, I, P, I, I, I, I, I, I, P],
    "hfa_qkv_prepare": [P, I, I, P, P, I, I, I, I, I, I, P, P, F, P, P, P, P, P, P, I, I, P],
    "hfa_causal_conv": [P, I, I, P, P, I, I, P, c_size_t, P, P, I, I, P, I, I, P],
    "hfa_linear_scan": [P, I, P, I, I, I, P, I, I, I, I, I, P, P, I, I, P, P, P, P, c_size_t, P, P, I, P, I, P, P, F, F, P, P],
    "hfa_moe_gated_act": [P, I, P, P, P, I, I, I, I, F, F, F, I, P],
    "hfa_rope_table": [P, P, I, P, I, P],
    "hfa_decode_attention_supports": [I, I, I, I, I, I, I, I],
    "hfa_decode_attention": [P, I, P, P, P, I, P, P, I, P, P, P, I, I, P, I, I, I, I, I, I, I, F, P, c_size_t, P],
    "hfa_layernorm": [P, P, P, P, I, P, I, I, F, P, I, P, I, P],
    "hfa_activation": [P, I, P, I, I, I, I, I, P],
    "hfa_softcap": [P, I, I, I, F, P],
    "hfa_moe_route": [P, I, I, I, I, I, I, I, I, F, P, P, P],
    "hfa_moe_plan": [P, I, I, I, P, P, P, P],
    "hfa_moe_gemm": [P, I, I, I, P, I, P, P, P, I, I, P, I, I, I, P, I, I, I, I, I, F, F, F, P],
    "hfa_moe_combine": [P, P, I, I, I, P],
    "hfa_swiglu": [P, P, I, I, I, P],
    "hfa_scatter_i32": [P, P, P, I, P],
    "hfa_move_i32": [P, P, P, P, I, P],
    "hfa_argmax": [P, I, P, I, I, P, c_size_t, P],
    "hfa_argmax_static": [P, I, P, I, I, P],
    "hfa_topk": [P, I, P, P, P, I, I, I, P],
    "hfa_order_rows": [P, I, P, P, P, I, I, P, c_size_t, P],
    "hfa_draw_rows": [P, P, I, I, P, P, P, P],
    "hfa_random_fill": [P, I, c_size_t, ctypes.c_uint64, F, I, I, P],
    "hfa_probe_read": [P, c_size_t, P, I, P],
    "hfa_probe_copy": [P, P, c_size_t, P],
    "hfa_probe_mfma": [P, I, I, P, P],
}


def library():
    """The loaded library (built first if there is none, or if its sources changed)."""
    global _lib
    with _lock:
        if _lib is None:
            path, current = _build.find_library()
            if path is None or not current:
                path = _build.build()
            lib = ctypes.CDLL(path)
            lib.hfa_last_error.restype = c_char_p
            lib.hfa_last_error.argtypes = []
            lib.hfa_version.restype = c_int
            lib.hfa_order_rows_scratch.restype = c_size_t
            lib.hfa_order_rows_scratch.argtypes = [c_int, c_int]
            lib.hfa_gemm_rows_parts.restype = c_int
            lib.hfa_gemm_rows_parts.argtypes = []
            lib.hfa_probe_mfma_threads.restype = c_int
            lib.hfa_probe_mfma_threads.argtypes = []
            lib.hfa_attention_prompt_rows.restype = c_int
            lib.hfa_attention_prompt_rows.argtypes = []
            lib.hfa_linear_scan_state_floats.restype = c_size_t
            lib.hfa_linear_scan_state_floats.argtypes = [c_int] * 3
            lib.hfa_linear_scan_max_floats.restype = c_size_t
            lib.hfa_linear_scan_max_floats.argtypes = [c_int] * 3
            lib.hfa_moe_tile_rows.restype = c_int
            lib.hfa_moe_tile_rows.argtypes = [c_int] * 6
            for name, args in _SIGNATURES.items():
                fn = getattr(lib, name)
                fn.argtypes = args
                fn.restype = c_int
            lib.path = path
            _lib = lib
        return _lib


def load_extension(path, signatures):
    """A shared library with kernels of a part that is not the package's: ``signatures`` maps each
    entry point to its ctypes argument types (the stream last; it returns an int, 0 = done).
    The part calls them through ``Ops.call``."""
    lib = ctypes.CDLL(path)
    for name, args in signatures.items():
        fn = getattr(lib, name)
        fn.argtypes = list(args)
        fn.restype = c_int
    lib.path = path
    return lib


def last_error():
    return library().hfa_last_error().decode("utf-8", "replace")
