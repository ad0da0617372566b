"""ctypes loader for oracle/libkvoracle.so (TEST INFRASTRUCTURE ONLY).

Wraps the scalar C restatement in kv_oracle.c; see that file's header for the
reference lines each function follows and for its parity status.
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "libkvoracle.so")
DT = {"float16": 0, "bfloat16": 1, "float32": 2}


def build(force: bool = False) -> str:
    src = os.path.join(_HERE, "kv_oracle.c")
    if force or not os.path.exists(_SO) or os.path.getmtime(_SO) < os.path.getmtime(src):
        subprocess.check_call(["make", "-C", _HERE, "-B", "libkvoracle.so"],
                              stdout=subprocess.DEVNULL)
    return _SO


class _Mask(C.Structure):
    _fields_ = [("mode", C.c_int32), ("bool_data", C.c_void_p), ("add_data", C.c_void_p),
                ("sb", C.c_int64), ("sh", C.c_int64), ("sl", C.c_int64)]


_lib = None


def lib():
    global _lib
    if _lib is None:
        _lib = C.CDLL(build())
        _lib.kvo_round.restype = C.c_float
        _lib.kvo_round.argtypes = [C.c_float, C.c_int]
        _lib.kvo_num_threads.restype = C.c_int
    return _lib


def _p(a):
    return a.ctypes.data_as(C.c_void_p)


def num_threads() -> int:
    return lib().kvo_num_threads()


def affine_quantize(w, group_size, bits, dtype):
    w = np.ascontiguousarray(w, np.float32)
    D = w.shape[-1]
    rows = w.size // D
    wq = np.empty(w.shape[:-1] + (D * bits // 32,), np.uint32)
    s = np.empty(w.shape[:-1] + (D // group_size,), np.float32)
    b = np.empty_like(s)
    lib().kvo_affine_quantize(_p(w), C.c_int64(rows), D, group_size, bits, DT[dtype], _p(wq), _p(s), _p(b))
    return wq, s, b


def affine_dequantize(wq, s, b, group_size, bits, dtype):
    wq = np.ascontiguousarray(wq, np.uint32)
    s = np.ascontiguousarray(s, np.float32)
    b = np.ascontiguousarray(b, np.float32)
    D = wq.shape[-1] * 32 // bits
    rows = wq.size // wq.shape[-1]
    out = np.empty(wq.shape[:-1] + (D,), np.float32)
    lib().kvo_affine_dequantize(_p(wq), _p(s), _p(b), C.c_int64(rows), D, group_size, bits, DT[dtype], _p(out))
    return out


def _mask_struct(mask, B, Hq, L, T, keep):
    """mask: None | "causal" | numpy array broadcastable to [B,Hq,L,T]."""
    if mask is None:
        return None
    m = _Mask()
    if isinstance(mask, str):
        assert mask == "causal"
        m.mode = 1
        return m
    a = np.asarray(mask)
    while a.ndim < 4:
        a = a[None]
    assert a.shape[-1] == T and a.shape[-2] == L
    sb = 0 if a.shape[0] == 1 else a.shape[1] * L * T
    sh = 0 if a.shape[1] == 1 else L * T
    if a.dtype == np.bool_:
        a = np.ascontiguousarray(a.astype(np.uint8))
        m.mode, m.bool_data = 2, a.ctypes.data
    else:
        a = np.ascontiguousarray(a, np.float32)
        m.mode, m.add_data = 3, a.ctypes.data
    keep.append(a)
    m.sb, m.sh, m.sl = sb, sh, T
    return m


def qsdpa(q, qkeys, qvalues, scale, mask, group_size, bits, dtype):
    q = np.ascontiguousarray(q, np.float32)
    kw, ks, kb = (np.ascontiguousarray(a) for a in qkeys)
    vw, vs, vb = (np.ascontiguousarray(a) for a in qvalues)
    B, Hq, L, Dk = q.shape
    Hkv, T = kw.shape[1], kw.shape[2]
    Dv = vw.shape[-1] * 32 // bits
    out = np.empty((B, Hq, L, Dv), np.float32)
    scratch = np.empty((B, Hq, L, T), np.float32)
    keep = []
    m = _mask_struct(mask, B, Hq, L, T, keep)
    lib().kvo_qsdpa(_p(q), _p(kw), _p(ks.astype(np.float32)), _p(kb.astype(np.float32)),
                    _p(vw), _p(vs.astype(np.float32)), _p(vb.astype(np.float32)),
                    B, Hq, Hkv, L, T, Dk, Dv, group_size, bits, DT[dtype], C.c_float(scale),
                    C.byref(m) if m is not None else None, _p(scratch), _p(out))
    return out


def sdpa(q, k, v, scale, mask, dtype):
    q = np.ascontiguousarray(q, np.float32)
    k = np.ascontiguousarray(k, np.float32)
    v = np.ascontiguousarray(v, np.float32)
    B, Hq, L, Dk = q.shape
    Hkv, T, Dv = k.shape[1], k.shape[2], v.shape[3]
    out = np.empty((B, Hq, L, Dv), np.float32)
    keep = []
    m = _mask_struct(mask, B, Hq, L, T, keep)
    lib().kvo_sdpa(_p(q), _p(k), _p(v), B, Hq, Hkv, L, T, Dk, Dv, DT[dtype], C.c_float(scale),
                   C.byref(m) if m is not None else None, _p(out))
    return out
