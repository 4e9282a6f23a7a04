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
                         c_int, c_int, c_float, c_int, c_int, c_float, c_void, c_int, c_int],
        "sp_attention_decode_project_takes": [c_int] * 7,
        "sp_attention_decode_project": [c_void, c_void, c_int, c_void, c_void, c_void, c_int, c_void, c_void, c_void,
                                        c_int, c_int, c_void, c_i64, c_void, c_void, c_int, c_int, c_int, c_int, c_int,
                                        c_int, c_int, c_float, c_int, c_float, c_void, c_int],
        "sp_attention_plan": [c_int, c_int, c_int, c_int, c_int, c_int, ctypes.POINTER(c_int)],
        "sp_fused_supported": [c_int] * 8,
        "sp_fused_norm_pays": [c_int] * 3,
        "sp_pipe_plan": [c_int, c_int, c_int, c_int, c_int, ctypes.POINTER(c_int)],
        "sp_pipe_tiles": [c_int, c_int, ctypes.POINTER(c_int), c_int],
        "sp_gemm_decode": [c_void, c_void, c_void, c_int, c_void, c_float, c_void, c_int, c_void, c_int, c_void, c_int,
                           c_int, c_int],
        "sp_qkv_rope_cache": [c_void, c_void, c_void, c_int, c_void, c_float, c_void, c_int, c_void, c_void, c_void,
                              c_void, c_int, c_void, c_void, c_void, c_int, c_int, c_int, c_int, c_int, c_int, c_void, c_int],
        "sp_rope_table": [c_void, c_void, c_void, c_void, c_int, c_float, c_void, c_int],
        "sp_scale": [c_void, c_void, c_float, c_i64],
        "sp_scaled_add": [c_void, c_void, c_void, c_int, c_void, c_float, c_void, c_void, c_float, c_int, c_int],
        "sp_head_gate": [c_void, c_int, c_void, c_void, c_i64, c_int, c_int, c_int],
        "sp_rglru_takes": [c_int] * 3,
        "sp_rglru": [c_void, c_int, c_void, c_i64, c_int, c_int, c_int, c_int, c_int] + [c_void] * 16 + [c_int, c_int, c_int, c_void],
        "sp_retention_takes": [c_int] * 2,
        "sp_retention": [c_void, c_int, c_void, c_i64, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_void, c_void,
                         c_float, c_void, c_void, c_void, c_void, c_void, c_int, c_int, c_int, c_void],
        "sp_gate_up_silu": [c_void, c_void, c_void, c_int, c_void, c_float, c_void, c_void, c_int, c_int, c_int, c_int, c_float, c_void, c_i64],
        "sp_gate_up_silu_f32_takes": [c_int, c_int, c_int],
        "sp_gate_up_silu_f32": [c_void, c_void, c_void, c_float, c_void, c_void, c_int, c_int, c_int, c_int, c_float, c_void, c_i64],
        "sp_qkv_rope_cache_f32_takes": [c_int] * 7,
        "sp_qkv_rope_cache_f32": [c_void, c_void, c_void, c_float, c_void, c_int, c_void, c_void, c_void, c_void, c_void,
                                  c_int, c_void, c_void, c_void, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_int],
        "sp_silu_mul": [c_void, c_int, c_void, c_void, c_int, c_int, c_int, c_float, c_void, c_i64],
        "sp_sample": [c_void, c_void, c_void, c_void, c_void, c_void, c_void, c_int, c_int],
        "sp_sample_workspace_floats": [c_int, c_int],
        "sp_feed_tokens": [c_void, c_void, c_void, c_void, c_int, c_int],
        "sp_random_fill": [c_void, c_int, c_void, c_i64, ctypes.c_uint64, c_i64, c_float, c_float, c_int],
        "sp_layernorm": [c_void, c_void, c_void, c_int, c_void, c_void, c_void, c_void, c_float, c_int, c_void, c_void, c_int, c_int],
        "sp_embed_bigram": [c_void, c_int, c_void, c_void, c_void, c_void, c_void, c_void, c_void, c_void, c_void, c_void,
                            c_int, c_int, c_int, c_i64, c_i64, c_i64],
        "sp_latent_prepare": [c_void, c_int, c_void, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_void, c_float,
                              c_void, c_void, c_int, c_float, c_int, c_void, c_void, c_void, c_int, c_int, c_void, c_int],
        "sp_head_gemm": [c_void, c_int, c_void, c_i64, c_i64, c_void, c_void, c_i64, c_i64, c_void, c_i64, c_int, c_int,
                         c_int, c_int],
        "sp_group_tile_rows": [c_int, c_i64, c_int, c_int],
        "sp_route_topk": [c_void, c_void, c_void, c_void, c_int, c_int, c_int],
        "sp_route_max_tiles": [c_int, c_int, c_int],
        "sp_route": [c_void, c_void, c_void, c_void, c_int, c_int, c_int, c_int, c_void, c_void, c_void, c_void],
        "sp_route_sort": [c_void, c_void, c_int, c_int, c_int, c_void, c_void, c_void, c_void],
        "sp_expert_gate_up": [c_void, c_int, c_void, c_void, c_void, c_void, c_int, c_int, c_void, c_int, c_void, c_int,
                              c_int, c_int, c_int, c_int, c_float],
        "sp_route_scored": [c_void, c_void, c_i64, c_void, c_int, c_int, c_float, c_void, c_void, c_int, c_int, c_int, c_int,
                            c_int, c_void, c_void, c_void, c_void],
        "sp_route_combine_identity": [c_void, c_void, c_void, c_void, c_int, c_void, c_int, c_void, c_int, c_void, c_int, c_int],
        "sp_qkv_prepare": [c_void, c_int, c_void, c_i64, c_int, c_int, c_int, c_int, c_int, c_void, c_void, c_float, c_void,
                           c_void, c_void, c_int, c_void, c_void, c_int, c_void, c_void, c_void, c_int, c_int, c_void, c_int,
                           c_float, c_int],
        "sp_expert_down": [c_void, c_int, c_void, c_void, c_void, c_void, c_int, c_int, c_void, c_int, c_int, c_int, c_int],
        "sp_route_combine": [c_void, c_void, c_void, c_void, c_int, c_void, c_int, c_int],
        "sp_route_sigmoid": [c_void, c_void, c_void, c_void, c_int, c_int, c_int, c_int, c_void, c_void, c_void, c_void],
        "sp_short_conv": [c_void, c_int, c_void, c_i64, c_int, c_int, c_int, c_int, c_void, c_void, c_int, c_int, c_void, c_i64,
                          c_int, c_void, c_void, c_void, c_void, c_void, c_int, c_int, c_int],
        "sp_group_rmsnorm": [c_void, c_void, c_int, c_void, c_float, c_int, c_void, c_int, c_int, c_int],
        "sp_activation": [c_void, c_int, c_void, c_i64, c_int],
        "sp_scale_rows": [c_void, c_int, c_void, c_void, c_int, c_void, c_int, c_int],
        "sp_ssd_scan": [c_void, c_int, c_void, c_i64, c_int, c_int, c_void, c_i64, c_int, c_int, c_int, c_int, c_void, c_void,
                        c_void, c_void, c_void, c_void, c_void, c_void, c_int, c_int, c_int, c_void],
        "sp_selective_scan": [c_void, c_int, c_void, c_i64, c_int, c_void, c_i64, c_int, c_void, c_void, c_i64, c_int, c_int,
                              c_int, c_void, c_void, c_void, c_void, c_void, c_void, c_void, c_int, c_int, c_int, c_void],
        "sp_qk_cross_prepare": [c_void, c_int, c_void, c_int, c_int, c_int, c_int, c_int, c_void, c_void, c_float, c_void,
                                c_void, c_int, c_void, c_void, c_void, c_void, c_int, c_int],
        "sp_head_mix": [c_void, c_int, c_void, c_void, c_int, c_int, c_int, c_int, c_void, c_int],
        "sp_probe_read": [c_void, c_void, c_i64, c_int, c_void],
        "sp_probe_mfma": [c_void, c_int, c_int, c_void, ctypes.POINTER(ctypes.c_double)],
    }
    lib.sp_attention_workspace_floats.argtypes = [c_int] * 10
    lib.sp_attention_workspace_floats.restype = c_i64
    lib.sp_rglru_carry_floats.argtypes = [c_int] * 4
    lib.sp_rglru_carry_floats.restype = c_i64
    lib.sp_retention_scratch_floats.argtypes = [c_int] * 6
    lib.sp_retention_scratch_floats.restype = c_i64
    lib.sp_ssd_scan_scratch_floats.argtypes = [c_int] * 5
    lib.sp_ssd_scan_scratch_floats.restype = c_i64
    lib.sp_selective_scan_scratch_floats.argtypes = [c_int] * 4
    lib.sp_selective_scan_scratch_floats.restype = c_i64
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
