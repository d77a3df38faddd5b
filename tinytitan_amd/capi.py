"""ctypes loader of libctinytitan_hip.so (the C ABI declared in include/ctinytitan_hip.h).

Loads the library that ``tinytitan_amd.build`` produced in-tree.  There is no
fallback of any kind: a missing library raises, and every entry point that
computes needs a gfx950 device.
"""
from __future__ import annotations

import ctypes
import os
import re
from typing import List

PKG = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.environ.get("TT_HIP_LIBRARY", os.path.join(PKG, "lib", "libctinytitan_hip.so"))  # override: a differently built copy
HEADER_PATH = os.path.join(os.path.dirname(PKG), "include", "ctinytitan_hip.h")

OK = 0
ERR_INVALID_ARGUMENT = 1
ERR_SHAPE = 2
ERR_CURSOR = 3
ERR_CAPACITY = 4
ERR_BUSY = 5
ERR_OUT_OF_MEMORY = 6
ERR_HIP = 7
ERR_NO_DEVICE = 8
ERR_STALE = 9
ERR_SCRATCH = 10

OPT_KV_STREAM = 1
OPT_XCD_GRID = 2
OPT_MEASURE_PASS_ONLY = 3

_c_int_p = ctypes.POINTER(ctypes.c_int)
_vp = ctypes.c_void_p
_i = ctypes.c_int
_sz = ctypes.c_size_t

_SIGNATURES = {
    "tt_hip_ctx_create": (_vp, [_i, _c_int_p]),
    "tt_hip_ctx_destroy": (None, [_vp]),
    "tt_hip_ctx_set_stream": (_i, [_vp, _vp]),
    "tt_hip_ctx_set_default_stream": (_i, [_vp]),
    "tt_hip_calibrate_read": (_i, [_vp, _vp, _sz, _vp, _vp]),
    "tt_hip_ctx_stream": (_vp, [_vp]),
    "tt_hip_sync": (_i, [_vp]),
    "tt_hip_timer_begin": (_i, [_vp]),
    "tt_hip_timer_end": (_i, [_vp, ctypes.POINTER(ctypes.c_uint64)]),
    "tt_hip_profile_enable": (_i, [_vp, _i]),
    "tt_hip_profile_disable": (_i, [_vp]),
    "tt_hip_profile_read": (_i, [_vp, _c_int_p, ctypes.POINTER(ctypes.c_uint64)]),
    "tt_hip_profile_event_overhead_ns": (_i, [_vp, ctypes.POINTER(ctypes.c_uint64)]),
    "tt_hip_graph_begin": (_i, [_vp]),
    "tt_hip_graph_end": (_i, [_vp, ctypes.POINTER(_vp)]),
    "tt_hip_graph_launch": (_i, [_vp, _vp]),
    "tt_hip_graph_destroy": (None, [_vp]),
    "tt_hip_split_geometry": (_i, [_vp, _i, _i, _i, _i, _i, _i, _c_int_p, _c_int_p, _c_int_p]),
    "tt_hip_set_split_tokens": (_i, [_vp, _i]),
    "tt_hip_set_option": (_i, [_vp, _i, _i]),
    "tt_hip_strerror": (ctypes.c_char_p, [_i]),
    "tt_hip_last_hip_error": (ctypes.c_char_p, [_vp]),
    "tt_hip_kv_create": (_vp, [_vp, _i, _i, _i, _i, _i, _i, _c_int_p]),
    "tt_hip_kv_create_quantized": (_vp, [_vp, _i, _i, _i, _i, _i, _i, _i, _c_int_p]),
    "tt_hip_kv_create_ring": (_vp, [_vp, _i, _i, _i, _i, _i, _i, _i, _c_int_p]),
    "tt_hip_kv_precision_bits": (_i, [_vp]),
    "tt_hip_kv_row_layout": (_i, [_i, _i, ctypes.POINTER(ctypes.c_size_t), ctypes.POINTER(ctypes.c_size_t)]),
    "tt_hip_kv_export_rows": (_i, [_vp, _i, _i, _i, _i, _vp, _vp, _sz]),
    "tt_hip_kv_import_rows": (_i, [_vp, _i, _i, _i, _i, _vp, _vp, _sz]),
    "tt_hip_kv_destroy": (None, [_vp]),
    "tt_hip_kv_capacity": (_i, [_vp]),
    "tt_hip_kv_max_context": (_i, [_vp]),
    "tt_hip_kv_position": (_i, [_vp, _i]),
    "tt_hip_kv_token_stride_bytes": (_sz, [_vp]),
    "tt_hip_kv_bytes": (_sz, [_vp]),
    "tt_hip_kv_append": (_i, [_vp, _i, _i, _i, _i, _vp, _vp, _sz]),
    "tt_hip_kv_read": (_i, [_vp, _i, _i, _i, _i, _vp, _vp, _sz]),
    "tt_hip_kv_gather": (_i, [_vp, _i, _i, _vp, _i, _vp, _vp, _sz]),
    "tt_hip_kv_advance": (_i, [_vp, _i, _i]),
    "tt_hip_kv_rewind": (_i, [_vp, _i, _i]),
    "tt_hip_kv_reset": (_i, [_vp, _i]),
    "tt_hip_kv_reserve": (_i, [_vp, _i]),
    "tt_hip_kv_expect_position": (_i, [_vp, _i, _i]),
    "tt_hip_kv_k_offset": (_sz, [_i, _i, _i]),
    "tt_hip_kv_v_offset": (_sz, [_i, _i, _i]),
    "tt_hip_attn_decode": (_i, [_vp, _vp, _i, _i, _c_int_p, _c_int_p, _i, _vp, _vp, ctypes.c_float, _vp]),
    "tt_hip_attn_decode_noalloc": (_i, [_vp, _vp, _i, _i, _c_int_p, _c_int_p, _i, _vp, _vp, ctypes.c_float, _vp]),
    "tt_hip_attn_prefill": (_i, [_vp, _vp, _i, _i, _i, _i, _i, _i, _vp, _sz, _vp, _sz, ctypes.c_float, _vp, _sz]),
    "tt_hip_attn_decode_swa": (_i, [_vp, _vp, _i, _i, _c_int_p, _c_int_p, _i, _i, _vp, _vp, ctypes.c_float, _vp]),
    "tt_hip_attn_decode_keep": (_i, [_vp, _vp, _i, _i, _c_int_p, _c_int_p, _vp, _sz, _i, _vp, _vp, ctypes.c_float, _vp]),
    "tt_hip_attn_prefill_keep": (_i, [_vp, _vp, _i, _i, _i, _i, _i, _vp, _sz, _i, _vp, _sz, _vp, _sz, ctypes.c_float, _vp, _sz]),
    "tt_hip_attn_decode_keep_indices": (_i, [_vp, _vp, _i, _i, _c_int_p, _c_int_p, _vp, _sz, _vp, _i, _vp, _vp, ctypes.c_float, _vp]),
    "tt_hip_attn_prefill_keep_indices": (_i, [_vp, _vp, _i, _i, _i, _i, _i, _vp, _sz, _vp, _i, _vp, _sz, _vp, _sz, ctypes.c_float, _vp,
                                              _sz]),
    "tt_hip_attn_prefill_swa": (_i, [_vp, _vp, _i, _i, _i, _i, _i, _i, _i, _vp, _sz, _vp, _sz, ctypes.c_float, _vp, _sz]),
    "tt_hip_attn_verify_swa": (_i, [_vp, _vp, _i, _i, _c_int_p, _c_int_p, _i, _i, _i, _vp, _vp, ctypes.c_float, _vp]),
    "tt_hip_attn_verify": (_i, [_vp, _vp, _i, _i, _c_int_p, _c_int_p, _i, _i, _vp, _vp, ctypes.c_float, _vp]),
    "tt_hip_kv_snapshot_segment_count": (_i, [_vp]),
    "tt_hip_kv_snapshot_segment_lengths": (_i, [_vp, _i, ctypes.POINTER(ctypes.c_size_t), _i]),
    "tt_hip_kv_snapshot_export": (_i, [_vp, ctypes.POINTER(ctypes.c_size_t), _i, _vp, _sz, ctypes.POINTER(ctypes.c_size_t)]),
    "tt_hip_kv_snapshot_restore": (_i, [_vp, _i, ctypes.POINTER(ctypes.c_size_t), _i, _vp, _sz,
                                        ctypes.POINTER(ctypes.c_size_t)]),
    "tt_hip_qkv_epilogue_append": (_i, [_vp, _vp, _i, _i, _c_int_p, _c_int_p, _i, _i, _vp, _sz, _vp, _vp, _sz, _vp, _vp,
                                        ctypes.c_float, _i, ctypes.c_float, _vp, _sz, _vp, _sz]),
    "tt_hip_affine_projection": (_i, [_vp, _i, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _sz, _sz]),
    "tt_hip_qsa_pool_blocks": (_i, [_vp, _vp, _vp, _i, _i, _i, _i, _i, _vp, ctypes.c_float, ctypes.c_float]),
    "tt_hip_qsa_norm_rope_rows": (_i, [_vp, _vp, _i, _i, _i, _vp, ctypes.c_float, ctypes.c_float, _i, _i]),
    "tt_hip_qsa_block_scores": (_i, [_vp, _vp, _vp, _vp, _sz, _i, _i, _i, _i]),
    "tt_hip_qsa_decode_scores": (_i, [_vp, _vp, _vp, _i, _i, _i, _vp, _vp, _i, _vp, _i, ctypes.c_float, ctypes.c_float, _vp]),
    "tt_hip_qsa_select": (_i, [_vp, _vp, _sz, _i, _i, _i, _i, _vp, _sz, _vp, _sz, _vp]),
}

_lib = None


class LibraryMissing(RuntimeError):
    pass


def declared_symbols() -> List[str]:
    """Every function the public header declares."""
    text = open(HEADER_PATH, "r", encoding="utf-8").read()
    return sorted(set(re.findall(r"TT_HIP_API[^;(]*?\b(tt_hip_\w+)\s*\(", text)))


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise LibraryMissing(
                f"{LIB_PATH} is not built; run `python -m tinytitan_amd.build` (needs hipcc). "
                "There is no CPU fallback for this path.")
        L = ctypes.CDLL(LIB_PATH)
        for name, (restype, argtypes) in _SIGNATURES.items():
            fn = getattr(L, name)
            fn.restype = restype
            fn.argtypes = argtypes
        _lib = L
    return _lib


def strerror(status: int) -> str:
    return lib().tt_hip_strerror(status).decode()


def int_array(values):
    arr = (ctypes.c_int * len(values))(*[int(v) for v in values])
    return arr
