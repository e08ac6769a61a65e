"""ctypes binding of csrc/libmlc_hip.so (the C ABI of include/mlc_hip.h)."""
from __future__ import annotations

import ctypes as C
import os

from .build import LIB_PATH, build_all, built_from_current_sources


class NativeLibraryError(RuntimeError):
    pass


_u32p = C.POINTER(C.c_uint32)
_sz = C.c_size_t
_vp = C.c_void_p

# name -> (restype, argtypes); mirrors include/mlc_hip.h one to one.
SIGNATURES = {
    "mlc_hip_available": (C.c_int, []),
    "mlc_hip_last_error": (C.c_char_p, []),
    "mlc_hip_alloc": (_vp, [_sz]),
    "mlc_hip_free": (None, [_vp]),
    "mlc_hip_cached": (_vp, [C.c_char_p, _sz]),
    "mlc_hip_upload": (C.c_int, [_vp, _vp, _sz, _sz]),
    "mlc_hip_download": (C.c_int, [_vp, _vp, _sz, _sz]),
    "mlc_hip_zero": (C.c_int, [_vp, _sz]),
    "mlc_hip_begin": (C.c_int, []),
    "mlc_hip_flush": (C.c_int, []),
    "mlc_hip_has_open_pass": (C.c_int, []),
    "mlc_hip_paged_attn_decode": (C.c_int, [_vp, _vp, _vp, _vp, _u32p, _sz, _u32p, _u32p, _u32p,
                                            _sz, _sz, _sz, _sz, _sz, C.c_int, C.c_int]),
    "mlc_hip_paged_attn_decode_noalloc": (C.c_int, [_vp, _vp, _vp, _vp, _vp, _sz, _u32p, _u32p, _u32p,
                                                    _sz, _sz, _sz, _sz, _sz, C.c_int, _vp]),
    "mlc_hip_scatter_kv_paged_batched_f16": (C.c_int, [_vp, _u32p, _u32p, _sz, _sz, _sz, _sz, _vp,
                                                       C.c_int]),
    "mlc_hip_scatter_kv_paged": (C.c_int, [_vp, _u32p, _sz, _sz, _sz, _sz, _sz, _sz, _vp, _sz]),
    "mlc_hip_gather_kv_pages": (C.c_int, [_vp, _u32p, _sz, _sz, _sz, _sz, _sz, _vp, _sz]),
    "mlc_hip_qkv_split_rope_cast": (C.c_int, [_vp] * 8 + [_sz] * 9 + [C.c_int]),
    "mlc_hip_qkv_split_rope_scatter": (C.c_int, [_vp] * 8 + [_u32p, _u32p] + [_sz] * 10 + [C.c_int]),
    "mlc_hip_rms_norm_batched": (C.c_int, [_vp, _vp, _sz, C.c_float, _sz, _sz, _vp, C.c_int]),
    "mlc_hip_add_batched": (C.c_int, [_vp, _vp, _vp, _sz, C.c_int]),
    "mlc_hip_silu_mul_batched": (C.c_int, [_vp, _vp, _vp, _sz, C.c_int]),
    "mlc_hip_gate_up_split_silu_mul": (C.c_int, [_vp, _vp, _vp, _vp, _sz, _sz, _sz, C.c_int]),
    "mlc_hip_matmul_q4_0_batched": (C.c_int, [C.c_char_p, _vp, _sz, _vp, _sz, _sz, _sz, _sz, C.c_uint32, _vp,
                                              C.c_int]),
    "mlc_hip_matmul_q6_k_batched": (C.c_int, [C.c_char_p, _vp, _sz, _vp, _sz, _sz, _sz, _sz, _vp, C.c_int]),
    "mlc_hip_paged_attn_prefill": (C.c_int, [_vp, _vp, _vp, _vp, _u32p, _sz, _u32p, _u32p, _u32p,
                                             _sz, _sz, _sz, _sz, _sz, _sz, C.c_int]),
    "mlc_hip_capture_begin": (C.c_int, []),
    "mlc_hip_capture_end": (C.c_int, []),
    "mlc_hip_captured_launches": (_sz, [C.c_int]),
    "mlc_hip_replay_update": (C.c_int, [C.c_int, _u32p, _sz, _u32p, _u32p, _u32p, _u32p, _u32p, _sz]),
    "mlc_hip_replay": (C.c_int, [C.c_int]),
    "mlc_hip_capture_release": (None, [C.c_int]),
    "mlc_hip_stream": (_vp, []),
    "mlc_hip_timer_start": (C.c_int, []),
    "mlc_hip_timer_stop": (C.c_float, []),
    "mlc_hip_last_decode_launches": (C.c_int, []),
    "mlc_hip_last_decode_work_items": (C.c_int, []),
    "mlc_hip_last_decode_kernel": (C.c_char_p, []),
    "mlc_hip_row_program_launches": (C.c_long, []),
    "mlc_hip_decode_table_uploads": (C.c_long, []),
    "mlc_hip_fused_kv_write_launches": (C.c_long, []),
    "mlc_hip_fused_matmul_rope_launches": (C.c_long, []),
    "mlc_hip_fused_matmul_silu_launches": (C.c_long, []),
    "mlc_hip_fused_matmul_silu_split_launches": (C.c_long, []),
    "mlc_hip_fused_decode_split_launches": (C.c_long, []),
    "mlc_hip_fused_matmul_norm_launches": (C.c_long, []),
    "mlc_hip_kv_writes_in_decode_launches": (C.c_long, []),
    "mlc_hip_set_option": (C.c_int, [C.c_char_p, C.c_long]),
}

_lib = None


def load(build_if_missing: bool = True) -> C.CDLL:
    """Loads the native library.  It is built first when no built file exists or when the
    built file does not come from the sources as they are now (a stale library would be
    tested silently otherwise); with build_if_missing=False that is an error instead."""
    global _lib
    if _lib is not None:
        return _lib
    if not built_from_current_sources():
        if not build_if_missing:
            raise NativeLibraryError(f"{LIB_PATH} is missing or older than its sources; "
                                     "run mlcompiler_amd/build.py")
        build_all()
    try:
        lib = C.CDLL(LIB_PATH)
    except OSError as exc:  # pragma: no cover
        raise NativeLibraryError(f"cannot load {LIB_PATH}: {exc}") from exc
    for name, (res, args) in SIGNATURES.items():
        fn = getattr(lib, name)
        fn.restype = res
        fn.argtypes = args
    _lib = lib
    return lib
