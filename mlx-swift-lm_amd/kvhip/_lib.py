"""ctypes binding of libkvhip.so (the C ABI declared in include/kvhip.h).

There is no CPU fallback: importing this module without the built library, or
calling into it without a gfx950 device, raises.
"""
from __future__ import annotations

import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libkvhip.so")

OK = 0
KIND_SIMPLE, KIND_ROTATING, KIND_QUANTIZED = 0, 1, 2
F16, BF16, F32, U32, BOOL = 0, 1, 2, 3, 4
MASK_NONE, MASK_CAUSAL, MASK_ARRAY, MASK_WINDOW = 0, 1, 2, 3


class KVHipError(RuntimeError):
    def __init__(self, status, message):
        super().__init__(f"kvhip status {status}: {message}")
        self.status = status


class Config(C.Structure):
    _fields_ = [("kind", C.c_int32), ("step", C.c_int32), ("max_size", C.c_int32),
                ("keep", C.c_int32), ("group_size", C.c_int32), ("bits", C.c_int32)]


class Mask(C.Structure):
    _fields_ = [("mode", C.c_int32), ("dtype", C.c_int32), ("data", C.c_void_p),
                ("stride_b", C.c_int64), ("stride_h", C.c_int64), ("stride_l", C.c_int64),
                ("key_len", C.c_int32), ("offset", C.c_int32), ("window", C.c_int32),
                ("lengths", C.c_void_p), ("left_pad", C.c_void_p)]


class Rope(C.Structure):
    _fields_ = [("dims", C.c_int32), ("traditional", C.c_int32), ("base", C.c_float), ("scale", C.c_float),
                ("freqs", C.c_void_p)]


class MaskPlan(C.Structure):
    _fields_ = [("mode", C.c_int32), ("rows", C.c_int32), ("cols", C.c_int32),
                ("offset", C.c_int32), ("window", C.c_int32), ("rolled", C.c_int32),
                ("roll_shift", C.c_int32), ("roll_window", C.c_int32)]


# name -> (restype, argtypes); every symbol include/kvhip.h declares
_P, _I32, _I64, _F = C.c_void_p, C.c_int32, C.c_int64, C.c_float
SIGNATURES = {
    "kvhip_version": (C.c_char_p, []),
    "kvhip_last_error_message": (C.c_char_p, []),
    "kvhip_init": (_I32, [_I32]),
    "kvhip_sync": (_I32, [_P]),
    "kvhip_set_kernel_policy": (None, [_I32]),
    "kvhip_last_attend_kernel": (_I32, []),
    "kvhip_profile_enable": (None, [_I32]),
    "kvhip_profile_read": (_I32, [C.POINTER(_I32), C.POINTER(C.c_double)]),
    "kvhip_cache_create": (_I32, [C.POINTER(Config), C.POINTER(_P)]),
    "kvhip_cache_free": (None, [_P]),
    "kvhip_cache_copy": (_I32, [_P, _P, C.POINTER(_P)]),
    "kvhip_cache_reserve": (_I32, [_P, _I32, _I32, _I32, _I32, _I32, _I64]),
    "kvhip_cache_offset": (_I64, [_P]),
    "kvhip_cache_idx": (_I64, [_P]),
    "kvhip_cache_max_size": (_I64, [_P]),
    "kvhip_cache_group_size": (_I32, [_P]),
    "kvhip_cache_bits": (_I32, [_P]),
    "kvhip_cache_capacity": (_I64, [_P]),
    "kvhip_cache_presented_length": (_I64, [_P]),
    "kvhip_cache_device_rows": (_I64, [_P]),
    "kvhip_cache_slot_span": (_I64, [_P]),
    "kvhip_cache_is_trimmable": (_I32, [_P, _I64]),
    "kvhip_cache_trim": (_I64, [_P, _I64]),
    "kvhip_cache_set_offset": (_I32, [_P, _I64]),
    "kvhip_cache_update": (_I32, [_P, _P, _P, _I32, _I32, _I32, _I32, _I32, _I32, _P]),
    "kvhip_rope_apply": (_I32, [C.POINTER(Rope), _P, _P, _I32, _I32, _I32, _I32, _I32, _I64, _P, _P]),
    "kvhip_cache_update_rope": (_I32, [_P, C.POINTER(Rope), _P, _P, _P, _I32, _I32, _I32, _I32, _I32, _I32, _P]),
    "kvhip_cache_fetch": (_I32, [_P, _P, _P, _P]),
    "kvhip_cache_attend": (_I32, [_P, _P, _I32, _I32, _I32, _I32, _F, C.POINTER(Mask), _P, _P]),
    "kvhip_cache_attend_static": (_I32, [_P, _P, _I32, _I32, _I32, _I32, _F, C.POINTER(Mask), _P, _P]),
    "kvhip_cache_update_attend": (_I32, [_P, _P, _P, _P, _I32, _I32, _I32, _I32, _I32, _I32, _I32, _F,
                                         C.POINTER(Mask), _P, _P]),
    "kvhip_cache_mask_plan": (_I32, [_P, _I32, _I32, _I32, C.POINTER(MaskPlan)]),
    "kvhip_mask_materialize": (_I32, [C.POINTER(MaskPlan), _P, _P]),
    "kvhip_cache_state_count": (_I32, [_P]),
    "kvhip_cache_state_desc": (_I32, [_P, _I32, C.POINTER(_I64 * 4), C.POINTER(_I32)]),
    "kvhip_cache_state_export": (_I32, [_P, _I32, _P, _P]),
    "kvhip_cache_state_import": (_I32, [_P, _I32, C.POINTER(_P), C.POINTER(_I64), C.POINTER(_I32), _P]),
    "kvhip_cache_meta_count": (_I32, [_P]),
    "kvhip_cache_meta_get": (_I32, [_P, _I32, C.c_char_p, _I32]),
    "kvhip_cache_meta_set": (_I32, [_P, _I32, C.POINTER(C.c_char_p)]),
    "kvhip_cache_stage_begin": (_I32, [_P]),
    "kvhip_cache_stage_is_open": (_I32, [_P]),
    "kvhip_cache_stage_count": (_I64, [_P]),
    "kvhip_cache_stage_fetch": (_I32, [_P, _P, _P, _P]),
    "kvhip_cache_stage_commit": (_I32, [_P, _I64, _P]),
    "kvhip_cache_logical_view": (_I32, [_P, _I64, C.POINTER(_I64), _P, _P, _P]),
    "kvhip_cache_to_quantized": (_I32, [_P, _I32, _I32, _P, C.POINTER(_P)]),
    "kvhip_cache_to_unquantized": (_I32, [_P, _P, C.POINTER(_P)]),
    "kvhip_resolved_group_size": (_I32, [_I32, _I32, _I32]),
    "kvhip_affine_quantize": (_I32, [_P, _I64, _I32, _I32, _I32, _I32, _P, _P, _P, _P]),
    "kvhip_affine_dequantize": (_I32, [_P, _P, _P, _I64, _I32, _I32, _I32, _I32, _P, _P]),
}

_lib = None


def load():
    """Load libkvhip.so and bind every declared symbol.  Raises if it is not built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise ImportError(
                f"{LIB_PATH} is missing: build it with `make -C mlx-swift-lm_amd/csrc` "
                "(there is no CPU fallback)")
        lib = C.CDLL(LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(lib, name)
            fn.restype = res
            fn.argtypes = args
        _lib = lib
    return _lib


def check(status):
    if status < 0:
        msg = load().kvhip_last_error_message()
        raise KVHipError(status, msg.decode() if msg else "?")
    return status


_inited = False


def init(device: int = 0):
    global _inited
    if not _inited:
        check(load().kvhip_init(device))
        _inited = True
