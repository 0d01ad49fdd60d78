"""ctypes loader for ``libarcq_hip.so`` (the C ABI declared in ``include/arcq_hip.h``).

There is deliberately no fallback: if the shared library has not been built,
every op raises, so a GPU run can never silently go through something else.
"""
from __future__ import annotations

import ctypes
import os
import threading

_PKG_DIR = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_PKG_DIR, "libarcq_hip.so")

ARCQ_F32 = 0
ARCQ_F16 = 1
ARCQ_STATIC_SCRATCH_BYTES = 40 * 1024 * 1024

_c_i64 = ctypes.c_int64
_c_int = ctypes.c_int
_c_ptr = ctypes.c_void_p
_c_f32 = ctypes.c_float

class LinearExArgs(ctypes.Structure):
    """``arcq_linear_ex_args`` of include/arcq_hip.h."""
    _fields_ = [("struct_size", ctypes.c_uint32),
                ("x_dtype", ctypes.c_int32), ("y_dtype", ctypes.c_int32), ("producer", ctypes.c_int32),
                ("activation", ctypes.c_int32), ("bits", ctypes.c_int32), ("group_size", ctypes.c_int32),
                ("ln_eps", ctypes.c_float),
                ("M", ctypes.c_int64), ("N", ctypes.c_int64), ("K", ctypes.c_int64),
                ("x", ctypes.c_void_p), ("ln_weight", ctypes.c_void_p), ("ln_bias", ctypes.c_void_p),
                ("a_thresholds", ctypes.c_void_p), ("a_codebook", ctypes.c_void_p), ("packed_w", ctypes.c_void_p),
                ("w_codebook", ctypes.c_void_p), ("w_center", ctypes.c_void_p), ("w_scale", ctypes.c_void_p),
                ("w_code_sum", ctypes.c_void_p), ("bias", ctypes.c_void_p), ("residual", ctypes.c_void_p),
                ("x_hat_ws", ctypes.c_void_p), ("w_hat_ws", ctypes.c_void_p), ("y", ctypes.c_void_p),
                ("next_a_thresholds", ctypes.c_void_p), ("next_a_codebook", ctypes.c_void_p)]


ARCQ_PRODUCER_NONE, ARCQ_PRODUCER_LAYERNORM, ARCQ_PRODUCER_XHAT = 0, 1, 2
ARCQ_ACT_NONE, ARCQ_ACT_GELU = 0, 1

# name -> argtypes, in the order of include/arcq_hip.h
_SIGNATURES = {
    "arcq_pack_codes": [_c_ptr, _c_ptr, _c_i64, _c_i64, _c_int, _c_ptr],
    "arcq_unpack_codes": [_c_ptr, _c_ptr, _c_i64, _c_i64, _c_int, _c_ptr],
    "arcq_unpack_codes_u8": [_c_ptr, _c_ptr, _c_i64, _c_i64, _c_int, _c_ptr],
    "arcq_act_quant": [_c_ptr, _c_int, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_int,
                       _c_i64, _c_i64, _c_int, _c_int, _c_f32, _c_ptr],
    "arcq_weight_dequant": [_c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_int, _c_i64, _c_i64, _c_int, _c_int,
                            _c_ptr],
    "arcq_linear_fused": [_c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_int,
                          _c_i64, _c_i64, _c_i64, _c_int, _c_int, _c_ptr],
    "arcq_linear_otf": [_c_ptr, _c_int, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr,
                        _c_ptr, _c_int, _c_i64, _c_i64, _c_i64, _c_int, _c_int, _c_ptr],
    "arcq_linear_fused_ws": [_c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_int,
                             _c_i64, _c_i64, _c_i64, _c_int, _c_int, _c_ptr],
    "arcq_linear_otf_ws": [_c_ptr, _c_int, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr,
                           _c_ptr, _c_ptr, _c_int, _c_i64, _c_i64, _c_i64, _c_int, _c_int, _c_ptr],
    "arcq_linear_otf_static": [_c_ptr, _c_int, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr,
                               _c_ptr, _c_int, _c_i64, _c_i64, _c_i64, _c_int, _c_int, _c_ptr],
    "arcq_linear_otf_ex": [ctypes.POINTER(LinearExArgs), _c_ptr],
    "arcq_xhat_layout": [_c_i64],
    "arcq_act_quant_blocked_ln": [_c_ptr, _c_int, _c_ptr, _c_ptr, _c_f32, _c_ptr, _c_ptr, _c_ptr, _c_i64, _c_i64, _c_int,
                                  _c_f32, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_i64, _c_ptr],
    "arcq_act_quant_blocked": [_c_ptr, _c_int, _c_ptr, _c_ptr, _c_ptr, _c_i64, _c_i64, _c_int, _c_f32, _c_ptr],
    "arcq_act_quant_fp8": [_c_ptr, _c_int, _c_ptr, _c_ptr, _c_ptr, _c_i64, _c_i64, _c_int, _c_f32, _c_ptr],
    "arcq_weight_dequant_fp8": [_c_ptr] * 6 + [_c_i64, _c_i64, _c_int, _c_int, _c_f32, _c_ptr],
    "arcq_act_quant_fp8_blocked": [_c_ptr, _c_int, _c_ptr, _c_ptr, _c_ptr, _c_i64, _c_i64, _c_int, _c_f32,
                                   _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_i64, _c_f32, _c_ptr],
    "arcq_linear_fp8_blocked": [_c_ptr, _c_ptr, _c_ptr, _c_f32, _c_ptr, _c_int, _c_i64, _c_i64, _c_i64, _c_ptr],
    "arcq_linear_otf_fp8": [_c_ptr, _c_int, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_f32,
                            _c_ptr, _c_ptr, _c_ptr, _c_int, _c_i64, _c_i64, _c_i64, _c_int, _c_ptr],
    "arcq_act_quant_blocked_with_weights": [_c_ptr, _c_int, _c_ptr, _c_ptr, _c_ptr, _c_i64, _c_i64, _c_int, _c_f32,
                                            _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_i64, _c_ptr],
    "arcq_linear_fused_blocked": [_c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_int, _c_ptr, _c_int,
                                  _c_i64, _c_i64, _c_i64, _c_int, _c_int, _c_ptr],
    "arcq_act_quant_patches": [_c_ptr, _c_int, _c_ptr, _c_ptr, _c_ptr, _c_i64, _c_i64, _c_i64, _c_i64, _c_i64, _c_int, _c_f32,
                               _c_int, _c_ptr],
    "arcq_patch_embed_fwd": [_c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_i64, _c_i64, _c_i64, _c_i64, _c_i64, _c_ptr],
    "arcq_attention_fwd": [_c_ptr, _c_ptr, _c_i64, _c_i64, _c_i64, _c_i64, _c_f32, _c_ptr],
    "arcq_linear_forward_packed": [_c_ptr] * 11 + [_c_i64, _c_i64, _c_i64, _c_int, _c_int, _c_int, _c_ptr],
    "arcq_linear_forward_u8": [_c_ptr] * 11 + [_c_i64, _c_i64, _c_i64, _c_int, _c_int, _c_ptr],
}
EXPORTED_SYMBOLS = ("arcq_version", "arcq_last_error", "arcq_reload_tuning", "arcq_linear_fused_kernel",
                    "arcq_linear_fused_ws_kernel", "arcq_linear_otf_ws_kernel", "arcq_rows_wait_timeouts",
                    "arcq_rows_counter_slot") + tuple(_SIGNATURES)

_lib = None
_lock = threading.Lock()


class ARCQLibraryMissing(ImportError):
    pass


def load() -> ctypes.CDLL:
    """Load the library once; raise if it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    with _lock:
        if _lib is None:
            if not os.path.exists(LIB_PATH):
                raise ARCQLibraryMissing(
                    f"ARCQ HIP library is not built ({LIB_PATH} missing). "
                    "Run `python -m arcq_vit_amd.build` (needs hipcc) first.")
            lib = ctypes.CDLL(LIB_PATH)
            lib.arcq_version.restype = _c_int
            lib.arcq_version.argtypes = []
            lib.arcq_last_error.restype = ctypes.c_char_p
            lib.arcq_last_error.argtypes = []
            lib.arcq_reload_tuning.restype = None
            lib.arcq_reload_tuning.argtypes = []
            lib.arcq_linear_fused_kernel.restype = ctypes.c_char_p
            lib.arcq_linear_fused_kernel.argtypes = [ctypes.c_int64, ctypes.c_int64, ctypes.c_int64]
            lib.arcq_linear_fused_ws_kernel.restype = ctypes.c_char_p
            lib.arcq_linear_fused_ws_kernel.argtypes = [ctypes.c_int64, ctypes.c_int64, ctypes.c_int64, ctypes.c_int]
            lib.arcq_linear_otf_ws_kernel.restype = ctypes.c_char_p
            lib.arcq_linear_otf_ws_kernel.argtypes = [ctypes.c_int64, ctypes.c_int64, ctypes.c_int64, ctypes.c_int]
            lib.arcq_rows_wait_timeouts.restype = ctypes.c_longlong
            lib.arcq_rows_wait_timeouts.argtypes = []
            lib.arcq_rows_counter_slot.restype = _c_int
            lib.arcq_rows_counter_slot.argtypes = [ctypes.POINTER(ctypes.c_void_p), _c_int, _c_ptr]
            for name, argtypes in _SIGNATURES.items():
                fn = getattr(lib, name)
                fn.restype = _c_int
                fn.argtypes = argtypes
            _lib = lib
    return _lib


def check(rc: int) -> None:
    """Raise ``RuntimeError`` for a non-zero return, as ``TORCH_CHECK`` does in the reference's
    host wrappers (e.g. EXT/arcq_activation_kernel.cu:194-202)."""
    if rc != 0:
        msg = load().arcq_last_error().decode("utf-8", "replace")
        raise RuntimeError(msg or f"libarcq_hip call failed with code {rc}")


def reload_tuning() -> None:
    """Make the library read its ``ARCQ_*`` tuning variables again (it reads them once per process)."""
    load().arcq_reload_tuning()
