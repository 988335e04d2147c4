"""ctypes binding of libtract_rocm.so (the C ABI in include/tract_rocm.h).

There is no CPU fallback: if the shared library is missing or a call fails, an
exception is raised.
"""
from __future__ import annotations

import ctypes as C
import os

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "libtract_rocm.so")

F32, F16, Q8_0, Q4_0 = 0, 1, 2, 3


class TractRocmError(RuntimeError):
    """A call into libtract_rocm.so returned KO (the analogue of a TractResult Err)."""


_lib = None

_sz, _vp, _i, _i64, _f = C.c_size_t, C.c_void_p, C.c_int, C.c_int64, C.c_float
_pi64 = C.POINTER(C.c_int64)

# name -> argtypes; every function returns int unless listed in _RESTYPES
SIGNATURES = {
    "trocm_init": [_i],
    "trocm_last_error": [],
    "trocm_device_info": [C.POINTER(_i), C.POINTER(_sz), C.c_char_p, _sz],
    "trocm_malloc": [C.POINTER(_vp), _sz],
    "trocm_free": [_vp],
    "trocm_h2d": [_vp, _vp, _sz, _vp],
    "trocm_d2h": [_vp, _vp, _sz, _vp],
    "trocm_memset": [_vp, _i, _sz, _vp],
    "trocm_stream_create": [C.POINTER(_vp)],
    "trocm_stream_destroy": [_vp],
    "trocm_stream_sync": [_vp],
    "trocm_device_sync": [],
    "trocm_event_create": [C.POINTER(_vp)],
    "trocm_event_destroy": [_vp],
    "trocm_event_record": [_vp, _vp],
    "trocm_event_elapsed_ms": [_vp, _vp, C.POINTER(_f)],
    "trocm_copy_nd": [_vp, _sz, _pi64, _vp, _sz, _pi64, _pi64, _i, _i, _vp],
    "trocm_kv_cache_create": [C.POINTER(_vp), _i, _i64, _i64, _i64],
    "trocm_kv_cache_create_in_pool": [C.POINTER(_vp), _vp, _i, _i64, _i64, _i64],
    "trocm_kv_pool_create": [C.POINTER(_vp), _sz],
    "trocm_kv_pool_destroy": [_vp],
    "trocm_kv_pool_stats": [_vp, C.POINTER(_sz), C.POINTER(_sz), C.POINTER(_sz), C.POINTER(_vp)],
    "trocm_kv_cache_destroy": [_vp],
    "trocm_kv_cache_len": [_vp, _pi64],
    "trocm_kv_cache_capacity": [_vp, _pi64],
    "trocm_kv_cache_reallocs": [_vp, _pi64],
    "trocm_kv_cache_reserve": [_vp, _i64, _vp],
    "trocm_kv_append": [_vp, _vp, _i, _pi64, _i64, _vp],
    "trocm_kv_append_pair": [_vp, _vp, _vp, _vp, _i, _pi64, _i64, _vp],
    "trocm_kv_cache_truncate": [_vp, _i64],
    "trocm_kv_export": [_vp, _vp, _vp],
    "trocm_kv_row_bytes": [_vp, C.POINTER(_sz)],
    "trocm_kv_cache_clone": [_vp, C.POINTER(_vp), _vp],
    "trocm_kv_cache_raw": [_vp, C.POINTER(_vp), C.POINTER(_vp), _pi64],
    "trocm_kv_import_blocks": [_vp, _vp, _i64, _vp],
    "trocm_dat_header_write": [_vp, _i, _i, _pi64, _sz],
    "trocm_dat_header_read": [_vp, C.POINTER(_i), C.POINTER(_i), _pi64, C.POINTER(_sz), C.POINTER(_i)],
    "trocm_dat_q4_0_legacy_to_gguf": [_vp, _sz],
    "trocm_q8_1_to_q8_0": [_vp, _vp, _sz],
    "trocm_q8_0_to_q8_1": [_vp, _vp, _sz],
    "trocm_block_quant": [_i, _vp, _i, _sz, _vp, _vp],
    "trocm_block_dequant": [_i, _vp, _sz, _vp, _i, _vp],
    "trocm_block_simulate_precision_loss": [_i, _vp, _vp, _i, _sz, _vp],
    "trocm_q4_0_weights_create": [C.POINTER(_vp), _vp, _i64, _i64, _i64, _vp],
    "trocm_q4_0_weights_destroy": [_vp],
    "trocm_q4_0_weights_shape": [_vp, _pi64, _pi64, _pi64],
    "trocm_q4_0_weights_export": [_vp, _vp, _vp],
    "trocm_q4_0_matvec": [_vp, _vp, _i, _i64, _i64, _vp, _vp],
    "trocm_release_unused": [_i],
    "trocm_launch_floor": [_i, _vp, _sz, _i, _i, _vp, _vp],
    "trocm_cast": [_vp, _i, _vp, _i, _sz, _vp],
    "trocm_apply_rope": [_vp, _vp, _vp, _vp, _i, _i, _pi64, _pi64, _pi64, _pi64, _vp],
    "trocm_rotate_half": [_vp, _vp, _i, _i, _pi64, _pi64, _pi64, _vp],
    "trocm_sdpa_workspace_bytes": [_i64, _i64, _i64, _i64, C.POINTER(_sz)],
    "trocm_sdpa_workspace_init": [_vp, _sz, _vp],
    "trocm_sdpa": [_vp, _vp, _vp, _vp, _vp, _i, _i64, _i64, _i64, _i64, _i64, _i64, _pi64, _i64, _i64, _f, _i,
                   _vp, _sz, _vp],
    "trocm_sdpa_cached": [_vp, _i, _i64, _i64, _vp, _vp, _vp, _f, _i, _vp, _sz, _vp],
    "trocm_sdpa_cached_noalloc": [_vp, _i, _i64, _i64, _vp, _vp, _vp, _f, _i, _vp],
    "trocm_kv_cache_create_window": [C.POINTER(_vp), _i, _i64, _i64, _i64, _i64],
    "trocm_kv_cache_window": [_vp, _pi64, _pi64],
    "trocm_window_kv_sdpa_eval": [_vp, _vp, _vp, _i, _i64, _i64, _pi64, _vp, _vp, _vp, _f, _vp, _sz, _vp],
    "trocm_inplace_kv_sdpa_eval": [_vp, _vp, _vp, _i, _i64, _i64, _pi64, _vp, _vp, _vp, _f, _i, _vp, _sz, _vp],
    "trocm_inplace_kv_sdpa_eval_ragged_rope": [_vp, _vp, _vp, _vp, _vp, _i, _i64, _i64, C.POINTER(_vp), C.POINTER(_vp), _vp, _f, _vp, _sz, _vp, _sz, _vp],
    "trocm_inplace_kv_sdpa_eval_rope": [_vp, _vp, _vp, _vp, _vp, _i64, _i, _i64, _i64, _vp, _vp, _vp, _f, _i, _vp, _sz, _vp, _sz, _vp],
    "trocm_inplace_kv_sdpa_eval_ragged": [_vp, _vp, _vp, _i, _i64, _i64, C.POINTER(_vp), C.POINTER(_vp), _vp, _f, _vp,
                                          _sz, _vp],
    "trocm_kivi_cache_create": [C.POINTER(_vp), _i, _i, _i64, _i64, _i64, _i64],
    "trocm_kivi_cache_destroy": [_vp],
    "trocm_kivi_cache_reset": [_vp, _vp],
    "trocm_kivi_cache_len": [_vp, _pi64],
    "trocm_kivi_cache_counts": [_vp, _pi64, _pi64, _pi64, _pi64],
    "trocm_kivi_cache_memory_bytes": [_vp, C.POINTER(_sz)],
    "trocm_kivi_cache_append": [_vp, _vp, _i, _i64, _vp],
    "trocm_kivi_cache_dequantize": [_vp, _vp, _i, _vp],
    "trocm_kivi_cache_export": [_vp, _i, _vp, C.POINTER(_sz), _vp],
    "trocm_kivi_cache_clone": [_vp, C.POINTER(_vp), _vp],
    "trocm_quantized_kv_sdpa_eval": [_vp, _vp, _vp, _i, _i64, _i64, _vp, _vp, _vp, _f, _vp, _sz, _vp],
    "trocm_sdpa_decode_ragged": [_vp, _i, _i64, _i64, C.POINTER(_vp), C.POINTER(_vp), _vp, _f, _vp, _sz, _vp],
}
_RESTYPES = {"trocm_last_error": C.c_char_p}


def load() -> C.CDLL:
    """dlopen the library and attach the signatures (no GPU needed for this)."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise TractRocmError(
                f"{LIB_PATH} is missing: build it with `python -m tract_amd.build` (needs hipcc); "
                "there is no CPU fallback")
        lib = C.CDLL(LIB_PATH)
        for name, args in SIGNATURES.items():
            fn = getattr(lib, name)
            fn.argtypes = args
            fn.restype = _RESTYPES.get(name, C.c_int)
        _lib = lib
    return _lib


def check(rc: int) -> None:
    if rc != 0:
        raise TractRocmError(load().trocm_last_error().decode("utf-8", "replace"))


def call(name: str, *args) -> None:
    check(getattr(load(), name)(*args))
