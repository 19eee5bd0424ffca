"""Loads libsprout_hip.so (building it at the first call) and declares its C interface."""
from __future__ import annotations

import ctypes
import threading

_lock = threading.Lock()
_lib = None


class KernelError(RuntimeError):
    """A kernel entry point refused its arguments or a launch failed."""


def _declare(lib):
    c_int, c_void, c_float, c_i64 = ctypes.c_int, ctypes.c_void_p, ctypes.c_float, ctypes.c_int64
    lib.sp_last_error.restype = ctypes.c_char_p
    lib.sp_version.restype = c_int
    sig = {
        "sp_embed": [c_void, c_int, c_void, c_void, c_void, c_int, c_int, c_int],
        "sp_rmsnorm": [c_void, c_void, c_void, c_int, c_void, c_float, c_int, c_void, c_int, c_int],
        "sp_gemm": [c_void, c_int, c_void, c_int, c_void, c_int, c_void, c_int, c_int, c_void, c_int, c_int, c_int],
        "sp_rope_cache": [c_void, c_int, c_void, c_void, c_void, c_void, c_int, c_void, c_void, c_void, c_int, c_int,
                          c_int, c_int, c_int, c_int, c_int],
        "sp_attention": [c_void, c_int, c_void, c_int, c_void, c_void, c_void, c_int, c_void, c_void, c_void, c_void,
                         c_int, c_int, c_int, c_int, c_void, c_int, c_int, c_void, c_i64, c_void, c_int, c_int, c_int, c_int,
                         c_int, c_int, c_float, c_int, c_int],
        "sp_attention_decode_project_takes": [c_int] * 7,
        "sp_attention_decode_project": [c_void, c_void, c_int, c_void, c_void, c_void, c_int, c_void, c_void, c_void,
                                        c_int, c_int, c_void, c_i64, c_void, c_void, c_int, c_int, c_int, c_int, c_int,
                                        c_int, c_int, c_float, c_int],
        "sp_attention_plan": [c_int, c_int, c_int, c_int, c_int, c_int, ctypes.POINTER(c_int)],
        "sp_fused_supported": [c_int] * 8,
        "sp_fused_norm_pays": [c_int] * 3,
        "sp_pipe_plan": [c_int, c_int, c_int, c_int, c_int, ctypes.POINTER(c_int)],
        "sp_pipe_tiles": [c_int, c_int, ctypes.POINTER(c_int), c_int],
        "sp_gemm_decode": [c_void, c_void, c_void, c_int, c_void, c_float, c_void, c_int, c_void, c_int, c_void, c_int,
                           c_int, c_int],
        "sp_qkv_rope_cache": [c_void, c_void, c_void, c_int, c_void, c_float, c_void, c_int, c_void, c_void, c_void,
                              c_void, c_int, c_void, c_void, c_void, c_int, c_int, c_int, c_int, c_int, c_int, c_void, c_int],
        "sp_rope_table": [c_void, c_void, c_void, c_int, c_void, c_int],
        "sp_gate_up_silu": [c_void, c_void, c_void, c_int, c_void, c_float, c_void, c_void, c_int, c_int, c_int, c_int],
        "sp_gate_up_silu_f32_takes": [c_int, c_int, c_int],
        "sp_gate_up_silu_f32": [c_void, c_void, c_void, c_float, c_void, c_void, c_int, c_int, c_int, c_int],
        "sp_qkv_rope_cache_f32_takes": [c_int] * 7,
        "sp_qkv_rope_cache_f32": [c_void, c_void, c_void, c_float, c_void, c_int, c_void, c_void, c_void, c_void, c_void,
                                  c_int, c_void, c_void, c_void, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_int],
        "sp_silu_mul": [c_void, c_int, c_void, c_void, c_int, c_int, c_int],
        "sp_sample": [c_void, c_void, c_void, c_void, c_void, c_void, c_void, c_int, c_int],
        "sp_sample_workspace_floats": [c_int, c_int],
        "sp_feed_tokens": [c_void, c_void, c_void, c_void, c_int, c_int],
        "sp_random_fill": [c_void, c_int, c_void, c_i64, ctypes.c_uint64, c_i64, c_float, c_float, c_int],
        "sp_probe_read": [c_void, c_void, c_i64, c_int, c_void],
        "sp_probe_mfma": [c_void, c_int, c_int, c_void, ctypes.POINTER(ctypes.c_double)],
    }
    lib.sp_attention_workspace_floats.argtypes = [c_int] * 10
    lib.sp_attention_workspace_floats.restype = c_i64
    for name, argtypes in sig.items():
        fn = getattr(lib, name)
        fn.argtypes = argtypes
        fn.restype = c_int


def library():
    """The loaded library.  There is no fallback: without it the engine cannot run."""
    global _lib
    if _lib is None:
        with _lock:
            if _lib is None:
                from ..csrc.build import ensure_built
                path = ensure_built()
                try:
                    lib = ctypes.CDLL(path)
                except OSError as e:
                    raise KernelError(f"Cannot load the HIP kernel library {path}: {e}") from None
                _declare(lib)
                _lib = lib
    return _lib


def check(rc: int) -> None:
    if rc != 0:
        raise KernelError(library().sp_last_error().decode(errors="replace"))
