"""Prompt-cache files round-trip through device caches in the reference's wire format
(KVCache.swift:1797-2249), with the cases of the reference's KVCacheTests.swift."""
import numpy as np
import pytest
import torch
from safetensors import safe_open
from safetensors.torch import save_file

import kvhip
from tests.util import np32

pytestmark = pytest.mark.gpu


def ones(shape, dtype=torch.bfloat16):
    return torch.ones(shape, dtype=dtype, device="cuda")


def test_cache_serialization_round_trip(tmp_path):
    # KVCacheTests.swift:190-225 (testCacheSerialization) for the three classes of this library
    caches = [kvhip.KVCacheSimple(), kvhip.RotatingKVCache(32), kvhip.QuantizedKVCache()]
    k, v = ones((1, 8, 32, 64)), ones((1, 8, 32, 64))
    caches[0].update(k, v, fetch=False)
    caches[1].update(k, v, fetch=False)
    caches[2].update_quantized(k, v, fetch=False)
    url = tmp_path / "cache.safetensors"
    kvhip.save_prompt_cache(url, caches, {"model": "test"})
    loaded, meta = kvhip.load_prompt_cache(url)
    assert meta == {"model": "test"} and len(loaded) == 3
    for a, b in zip(caches, loaded):
        assert type(a) is type(b) and a.meta_state == b.meta_state and a.offset == b.offset
        sa, sb = a.state, b.state
        assert len(sa) == len(sb)
        for x, y in zip(sa, sb):
            assert x.shape == y.shape and x.dtype == y.dtype and torch.equal(x, y)
    # the file itself: Python-compatible class name, uint32 codes, metaState strings
    with safe_open(str(url), "pt") as f:
        md = f.metadata()
        assert md["2.0"] == "KVCache" and md["2.1"] == "RotatingKVCache" and md["2.2"] == "QuantizedKVCache"
        assert md["0.0.0"] == "" and [md[f"0.2.{j}"] for j in range(4)] == ["256", "32", "64", "8"]
        assert [md[f"0.1.{j}"] for j in range(6)] == ["0", "32", "256", "32", "32", "modelNative"]
        assert f.get_tensor("2.0").dtype == torch.uint32 and tuple(f.get_tensor("2.0").shape) == (1, 8, 32, 16)
        assert f.get_tensor("2.1").dtype == torch.bfloat16 and tuple(f.get_tensor("2.1").shape) == (1, 8, 32, 1)
        assert tuple(f.get_tensor("0.0").shape) == (1, 8, 32, 64)
    # a restored cache keeps working
    q = ones((1, 8, 1, 64))
    for a, b in zip(caches, loaded):
        oa = a.update_attend(q, k[:, :, :1], v[:, :, :1], 0.125)
        ob = b.update_attend(q, k[:, :, :1], v[:, :, :1], 0.125)
        assert torch.equal(oa, ob) and a.offset == b.offset == 33


def test_round_trip_preserves_empty_caches(tmp_path):
    # KVCacheTests.swift:608-638
    populated = kvhip.KVCacheSimple()
    populated.state = [ones((1, 1, 1, 32), torch.float32), ones((1, 1, 1, 32), torch.float32)]
    caches = [kvhip.KVCacheSimple(), populated, kvhip.RotatingKVCache(32), kvhip.QuantizedKVCache()]
    url = tmp_path / "empty.safetensors"
    kvhip.save_prompt_cache(url, caches)
    restored, _ = kvhip.load_prompt_cache(url)
    assert [type(c) for c in restored] == [type(c) for c in caches]
    assert restored[0].state == [] and len(restored[1].state) == 2 and restored[1].offset == 1
    assert restored[2].state == [] and restored[3].state == []


def test_quantized_group_size_fallback_survives_the_file(tmp_path):
    # KVCacheTests.swift:477-501: D = 32 lowers the group size to 32; a reload keeps it
    c = kvhip.QuantizedKVCache(64, 4)
    c.update_quantized(ones((1, 1, 4, 32)), ones((1, 1, 4, 32)), fetch=False)
    assert c.group_size == 32 and c.bits == 4
    url = tmp_path / "q.safetensors"
    kvhip.save_prompt_cache(url, [c])
    (r,), _ = kvhip.load_prompt_cache(url)
    assert r.group_size == 32 and r.bits == 4 and r.meta_state == c.meta_state
    r.update_quantized(torch.zeros((1, 1, 1, 32), dtype=torch.bfloat16, device="cuda"),
                       torch.zeros((1, 1, 1, 32), dtype=torch.bfloat16, device="cuda"), fetch=False)
    assert r.group_size == 32 and r.offset == 5


@pytest.mark.parametrize("bits", [3, 5, 6])
def test_code_widths_that_do_not_divide_32_survive_the_file(tmp_path, bits):
    # the packed arrays are [.., D * bits / 32] uint32 words of a bit stream; restore order: state, then metaState
    g = torch.Generator(device="cuda")
    g.manual_seed(bits)
    c = kvhip.QuantizedKVCache(32, bits)
    k = torch.randn(2, 2, 70, 96, generator=g, device="cuda").half()
    c.update_quantized(k, k.flip(-1), fetch=False)
    assert tuple(c.state[0].shape) == (2, 2, 70, 96 * bits // 32)
    url = tmp_path / "q.safetensors"
    kvhip.save_prompt_cache(url, [c])
    (r,), _ = kvhip.load_prompt_cache(url)
    assert r.bits == bits and r.group_size == 32 and r.offset == 70 and r.meta_state == c.meta_state
    for a, b in zip(r.state, c.state):
        assert torch.equal(a, b)
    q = torch.randn(2, 4, 1, 96, generator=g, device="cuda").half()
    assert torch.equal(r.attend(q, 96 ** -0.5), c.attend(q, 96 ** -0.5))


def write_fixture(path, class_name, array_count, metadata, shape=(1, 1, 1, 1)):
    # the fixture writer of KVCacheTests.swift:31-46
    arrays = {f"0.{i}": torch.zeros(shape, dtype=torch.float32) for i in range(array_count)}
    md = {f"0.0.{j}": v for j, v in enumerate(metadata)}
    md["2.0"] = class_name
    if not arrays:
        arrays = {}
    save_file(arrays, str(path), metadata=md)


def test_files_in_the_reference_layout(tmp_path):
    # KVCacheTests.swift:592-606: legacy 5-value rotating metadata gains the default origin
    url = tmp_path / "legacy.safetensors"
    write_fixture(url, "RotatingKVCache", 2, ["0", "32", "256", "1", "1"])
    (r,), _ = kvhip.load_prompt_cache(url)
    assert isinstance(r, kvhip.RotatingKVCache)
    assert r.meta_state == ["0", "32", "256", "1", "1", "modelNative"]
    # :551-590: incomplete state, invalid metadata, invalid rank
    bad = [("KVCacheSimple", 1, [""], (1, 1, 1, 1)),
           ("QuantizedKVCache", 3, ["256", "0", "64", "4"], (1, 1, 1, 1)),
           ("RotatingKVCache", 2, ["0", "32", "256", "0", "0", "invalid-origin"], (1, 1, 1, 1)),
           ("KVCacheSimple", 2, [""], (1, 1))]
    for i, (name, n, md, shape) in enumerate(bad):
        url = tmp_path / f"bad{i}.safetensors"
        write_fixture(url, name, n, md, shape)
        with pytest.raises(kvhip.KVCacheError):
            kvhip.load_prompt_cache(url)


def test_rotating_ring_state_survives_the_file(tmp_path):
    # a wrapped ring with a pinned prefix: the file keeps ring order and idx, and the restored
    # ring continues exactly like the original
    a = kvhip.RotatingKVCache(16, keep=2)
    rng = np.random.default_rng(0)
    def kv(n):
        t = torch.from_numpy(rng.standard_normal((1, 2, n, 64)).astype(np.float32)).to(torch.float16).cuda()
        return t, -t
    a.update(*kv(9), fetch=False)
    for _ in range(21):
        a.update(*kv(1), fetch=False)
    url = tmp_path / "ring.safetensors"
    kvhip.save_prompt_cache(url, [a])
    (b,), _ = kvhip.load_prompt_cache(url)
    assert b.meta_state == a.meta_state and b.idx == a.idx
    for _ in range(5):
        k, v = kv(1)
        ka, va = a.update(k, v)
        kb, vb = b.update(k, v)
        assert torch.equal(ka, kb) and torch.equal(va, vb)
    la, lb = a.logical_view(16), b.logical_view(16)
    assert torch.equal(la[0], lb[0]) and np.array_equal(np32(la[1]), np32(lb[1]))
