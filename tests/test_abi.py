"""CPU-side checks of the C ABI: the library loads, exports every symbol the
header declares, and the host bookkeeping (no device work) answers the integer
known answers of the reference's tests."""
import ctypes as C
import os
import re

import pytest

import kvhip
from kvhip import _lib as L

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "kvhip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(kvhip_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    lib = kvhip.load()
    names = declared_symbols()
    assert len(names) >= 35
    for n in names:
        assert hasattr(lib, n), f"{n} declared in kvhip.h but not exported"
    assert sorted(L.SIGNATURES) == names, "python binding and header disagree"
    assert b"gfx950" in lib.kvhip_version()


def make(kind, **kw):
    lib = kvhip.load()
    cfg = L.Config(kind=kind, step=kw.get("step", 0), max_size=kw.get("max_size", 0), keep=kw.get("keep", 0),
                   group_size=kw.get("group_size", 0), bits=kw.get("bits", 0))
    h = C.c_void_p()
    assert lib.kvhip_cache_create(C.byref(cfg), C.byref(h)) == 0
    return lib, h


def meta(lib, h):
    buf = C.create_string_buffer(64)
    out = []
    for i in range(lib.kvhip_cache_meta_count(h)):
        assert lib.kvhip_cache_meta_get(h, i, buf, 64) >= 0
        out.append(buf.value.decode())
    return out


def set_meta(lib, h, vals):
    arr = (C.c_char_p * len(vals))(*[v.encode() for v in vals])
    return lib.kvhip_cache_meta_set(h, len(vals), arr)


def test_rotating_trimmable_prediction():
    # KVCacheTests.swift:136-154
    lib, h = make(L.KIND_ROTATING, max_size=8)
    lib.kvhip_cache_set_offset(h, 3)
    assert lib.kvhip_cache_is_trimmable(h, 4) == 1 and lib.kvhip_cache_is_trimmable(h, 5) == 0
    for off in (8, 9):
        lib.kvhip_cache_set_offset(h, off)
        assert lib.kvhip_cache_is_trimmable(h, 0) == 0
    lib.kvhip_cache_free(h)


def test_quantized_meta_state():
    # KVCacheTests.swift:503-512
    lib, h = make(L.KIND_QUANTIZED, group_size=64, bits=8)
    assert meta(lib, h) == ["256", "0", "64", "8"]
    assert set_meta(lib, h, ["256", "11", "32", "4"]) == 0
    assert lib.kvhip_cache_offset(h) == 11 and lib.kvhip_cache_group_size(h) == 32 and lib.kvhip_cache_bits(h) == 4
    assert meta(lib, h) == ["256", "11", "32", "4"]
    assert set_meta(lib, h, ["256", "x", "32", "4"]) == L.OK - 4
    assert set_meta(lib, h, ["256", "1", "32"]) == L.OK - 4
    lib.kvhip_cache_free(h)


def test_rotating_meta_state():
    # KVCache.swift:775-815; legacy 5-field form KVCacheTests.swift:553-603
    lib, h = make(L.KIND_ROTATING, max_size=16, keep=2, step=128)
    assert meta(lib, h) == ["2", "16", "128", "0", "0", "modelNative"]
    assert set_meta(lib, h, ["0", "32", "256", "3", "3"]) == 0
    assert meta(lib, h) == ["0", "32", "256", "3", "3", "modelNative"]
    assert set_meta(lib, h, ["0", "32", "256", "3", "3", "requested"]) == 0
    assert meta(lib, h)[5] == "requested"
    assert set_meta(lib, h, ["0", "32", "256", "3", "3", "bogus"]) < 0
    assert b"capacity origin" in lib.kvhip_last_error_message()
    assert set_meta(lib, h, ["0", "None", "256", "3", "3"]) < 0
    assert set_meta(lib, h, ["0", "32", "256", "3"]) < 0
    lib.kvhip_cache_free(h)


def test_simple_meta_and_trim():
    lib, h = make(L.KIND_SIMPLE)
    assert meta(lib, h) == [""]
    assert set_meta(lib, h, [""]) == 0 and set_meta(lib, h, ["x"]) < 0
    lib.kvhip_cache_set_offset(h, 4)
    assert lib.kvhip_cache_trim(h, 3) == 3 and lib.kvhip_cache_offset(h) == 1
    assert lib.kvhip_cache_trim(h, 5) == 1 and lib.kvhip_cache_offset(h) == 0
    assert lib.kvhip_cache_max_size(h) == -1 and lib.kvhip_cache_is_trimmable(h, 100) == 1
    lib.kvhip_cache_free(h)


def test_group_size_resolution():
    # KVCache.swift:902-920, KVCacheTests.swift:477-484, Gemma4TextTests.swift:18-21
    lib = kvhip.load()
    assert lib.kvhip_resolved_group_size(64, 32, 32) == 32
    assert lib.kvhip_resolved_group_size(64, 128, 128) == 64
    assert lib.kvhip_resolved_group_size(64, 5, 5) == 0
    assert lib.kvhip_resolved_group_size(48, 128, 128) == 32
    assert lib.kvhip_resolved_group_size(64, 128, 96) == 32
    assert lib.kvhip_resolved_group_size(0, 256, 256) == 32


def plan(lib, h, n, window=0, return_array=0):
    p = L.MaskPlan()
    assert lib.kvhip_cache_mask_plan(h, n, window, return_array, C.byref(p)) == 0
    return p


def test_mask_plans_match_reference_mode_choice():
    # KVCacheTests.swift:816-848 and KVCache.swift:834-871
    lib, h = make(L.KIND_SIMPLE)
    assert plan(lib, h, 3).mode == L.MASK_CAUSAL and plan(lib, h, 1).mode == L.MASK_NONE
    lib.kvhip_cache_set_offset(h, 2)
    p = plan(lib, h, 3, return_array=1)
    assert (p.mode, p.rows, p.cols, p.offset, p.window) == (L.MASK_ARRAY, 3, 5, 2, 0)
    p = plan(lib, h, 5, window=4)
    assert (p.mode, p.rows, p.cols, p.window) == (L.MASK_ARRAY, 5, 7, 4)
    lib.kvhip_cache_free(h)
    lib, h = make(L.KIND_ROTATING, max_size=8)
    lib.kvhip_cache_set_offset(h, 20)
    p = plan(lib, h, 4, window=8)
    assert (p.mode, p.rows, p.cols, p.offset, p.window) == (L.MASK_ARRAY, 4, 11, 7, 8)
    assert plan(lib, h, 1).mode == L.MASK_NONE
    lib.kvhip_cache_set_offset(h, 2)
    assert plan(lib, h, 3).mode == L.MASK_CAUSAL
    lib.kvhip_cache_free(h)
    # rolled single-token window mask (window < maxSize, cache wrapped)
    lib, h = make(L.KIND_ROTATING, max_size=16)
    assert set_meta(lib, h, ["0", "16", "256", "21", "5"]) == 0
    p = plan(lib, h, 1, window=8)
    assert (p.mode, p.rolled, p.cols, p.roll_shift, p.roll_window) == (L.MASK_ARRAY, 1, 16, 6, 8)
    lib.kvhip_cache_free(h)


def test_errors_without_device_are_loud():
    lib, h = make(L.KIND_QUANTIZED, group_size=64, bits=4)
    assert lib.kvhip_cache_fetch(h, None, None, None) < 0
    assert b"updateQuantized" in lib.kvhip_last_error_message()
    assert lib.kvhip_cache_attend(h, None, 1, 1, 1, 1, C.c_float(1.0), None, None, None) < 0
    lib.kvhip_cache_free(h)
    lib.kvhip_cache_free(None)
    bad = L.Config(kind=7)
    out = C.c_void_p()
    assert lib.kvhip_cache_create(C.byref(bad), C.byref(out)) < 0
    rot = L.Config(kind=L.KIND_ROTATING, max_size=0)
    assert lib.kvhip_cache_create(C.byref(rot), C.byref(out)) < 0
