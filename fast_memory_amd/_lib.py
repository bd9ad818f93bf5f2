"""ctypes binding of libfastmem.so (the C ABI declared in include/fastmem.h).

There is no fallback: if the library is missing or does not load, every
operator of the package raises.
"""
from __future__ import annotations

import ctypes
import os
from ctypes import c_char_p, c_float, c_int, c_int32, c_int64, c_size_t, c_void_p

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libfastmem.so")

FM_F32, FM_BF16, FM_F16 = 0, 1, 2
FM_MAX_Z = 16384
FM_MAX_D = 256
FM_QTILE = 64
FM_STATIC_SCRATCH_BYTES = 32 << 20
FM_FUSED_STATUS_INTS = 66

P = c_void_p

# name -> (restype, argtypes); every symbol include/fastmem.h declares
SIGNATURES = {
    "fm_version": (c_int, []),
    "fm_last_error": (c_char_p, []),
    "fm_project": (c_int, [P, P, P, c_int, c_int, c_int, c_int, c_int64, c_int, P]),
    "fm_argtopz_workspace": (c_size_t, [c_int64, c_int, c_int]),
    "fm_argtopz_f32": (c_int, [P, c_int64, c_int, c_int64, c_int, P, P, P, c_size_t, P]),
    "fm_build_index_workspace": (c_size_t, [c_int, c_int, c_int, c_int, c_int, c_int64]),
    "fm_build_index": (c_int, [P, P, P, P, c_int, c_int, c_int, c_int, c_int, c_int, P, c_size_t, P]),
    "fm_build_index_fused_workspace": (c_size_t, [c_int, c_int, c_int, c_int, c_int, c_int]),
    "fm_build_index_fused": (c_int, [P, P, P, P, c_int, c_int, c_int, c_int, c_int, c_int, P, c_size_t, P, P]),
    "fm_qhash": (c_int, [P, P, P, P, c_int, c_int, c_int, c_int, c_int, P]),
    "fm_window_filter_workspace": (c_size_t, [c_int64]),
    "fm_window_filter": (c_int, [P, c_int64, c_int, c_int64, c_int64, P, P, P, P, c_size_t, P]),
    "fm_bucket_offsets": (c_int, [P, c_int64, P, P]),
    "fm_group_max_items": (c_int64, [c_int, c_int, c_int]),
    "fm_group_queries_workspace": (c_size_t, [c_int, c_int, c_int]),
    "fm_group_queries": (c_int, [P, c_int, c_int, c_int, P, P, P, P, P, c_int64, P, c_size_t, P]),
    "fm_hash_attn_fwd": (c_int, [P, P, P, P, P, P, P, P, P, c_int64, P, P, c_int, c_int, c_int, c_int,
                                 c_int, c_float, c_int, P]),
    "fm_hash_attn_fwd_workspace": (c_size_t, [c_int64]),
    "fm_debug_wave_pace_state": (c_int, [c_int, c_int, c_int, c_void_p, c_int, c_void_p]),
    "fm_hash_attn_fwd_ws": (c_int, [P, P, P, P, P, P, P, P, P, c_int64, P, P, c_int, c_int, c_int, c_int,
                                    c_int, c_float, c_int, P, c_size_t, P]),
    "fm_lists_key_order": (c_int, [P, P, P, c_int64, c_int, P, P, P]),
    "fm_hash_attn_bwd": (c_int, [P, P, P, P, P, P, P, P, P, c_int64, P, P, P, P, P, P, P, c_int, c_int, c_int, c_int,
                                 c_int, c_float, c_int, P]),
    "fm_inverse_index_workspace": (c_size_t, [c_int64, c_int, c_int]),
    "fm_inverse_index": (c_int, [P, P, P, c_int, c_int, c_int, c_int64, P, P, P, c_size_t, P]),
    "fm_inverse_index_key_order_workspace": (c_size_t, [c_int, c_int, c_int]),
    "fm_inverse_index_key_order": (c_int, [P, P, P, c_int, c_int, c_int, c_int64, P, P, P, P, c_size_t, P]),
    "fm_hash_attn_bwd_staged_workspace": (c_size_t, [c_int64]),
    "fm_hash_attn_bwd_staged": (c_int, [P, P, P, P, P, P, P, P, P, P, P, P, P, P, P, P, P, P, c_int, c_int, c_int,
                                        c_int, c_int, P, c_float, c_int, P, c_size_t, P]),
    "fm_attention_hash_varlen_workspace": (c_size_t, [c_int, c_int, c_int]),
    "fm_attention_hash_varlen": (c_int, [P, P, P, P, P, P, P, P, c_int, c_int, c_int, c_int, c_int,
                                         c_float, c_int, P, c_size_t, P]),
    "fm_attention_hash_varlen_static": (c_int, [P, P, P, P, P, P, P, P, c_int, c_int, c_int, c_int, c_int,
                                                c_float, c_int, P]),
    "fm_decode_hash_attn": (c_int, [P, P, P, P, P, P, c_int, c_int, c_int, c_float, P, P, P, P, c_int, P]),
    "fm_local_attn_fwd": (c_int, [P, P, P, P, P, c_int, c_int, c_int, c_int, c_int, c_float, c_int,
                                  c_int, P]),
    "fm_lse_merge": (c_int, [P, P, P, P, c_int64, c_int, c_int, P]),
    "fm_l2_normalize": (c_int, [P, P, c_int64, c_int, c_float, c_int, P]),
    "fm_topk_mean": (c_int, [P, P, P, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_int, P]),
    "fm_segment_mean": (c_int, [P, P, P, P, P, P, c_int, c_int, c_int, c_int, c_int, P]),
    "fm_segment_mean_directions": (c_int, [P, P, P, P, P, P, c_int, c_int, c_int, c_int, c_float, c_int, P]),
    "fm_index_append_workspace": (c_size_t, [c_int, c_int, c_int]),
    "fm_index_append": (c_int, [P, P, c_int, c_int, P, P, P, P, c_int, c_int, c_int, c_int, c_int, P, c_size_t, P, P]),
    "fm_segment_sum": (c_int, [P, P, P, P, P, c_int, c_int, c_int, c_int, c_int, P]),
    "fm_debug_hooks_enabled": (c_int, []),
    "fm_debug_force_generic": (None, [c_int]),
    "fm_hash_attn_fwd_kernel": (ctypes.c_char_p, [c_int] * 6),
    "fm_local_attn_fwd_kernel": (ctypes.c_char_p, [c_int] * 5),
    "fm_hash_attn_fwd_launches": (c_int, [c_int] * 6),
    "fm_build_index_fused_kernel": (ctypes.c_char_p, [c_int] * 6),
    "fm_debug_argtopz_exact_only": (None, [c_int]),
    "fm_debug_copy": (c_int, [P, P, c_int64, P]),
    "fm_debug_read": (c_int, [P, c_int64, P, P]),
    "fm_debug_gather": (c_int, [P, c_int64, c_int, P, P]),
    "fm_debug_fused_filter": (None, [c_int]),
    "fm_debug_mfma": (c_int, [P, c_int64, c_int, P, P]),
    "fm_debug_set_phase_events": (None, [P, c_int]),
}

_lib = None


def load() -> ctypes.CDLL:
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise RuntimeError(
            f"{LIB_PATH} is missing: build it with `python -m fast_memory_amd.build` "
            "(hipcc, --offload-arch=gfx950). There is no CPU or PyTorch fallback.")
    lib = ctypes.CDLL(LIB_PATH)
    for name, (res, args) in SIGNATURES.items():
        fn = getattr(lib, name)  # AttributeError if the library lacks a declared symbol
        fn.restype = res
        fn.argtypes = args
    _lib = lib
    return lib


class FastMemError(RuntimeError):
    pass


def check(rc: int) -> None:
    if rc == 0:
        return
    msg = load().fm_last_error().decode("utf-8", "replace")
    if rc == 1:
        raise ValueError(msg)
    raise FastMemError(f"libfastmem status {rc}: {msg}")
