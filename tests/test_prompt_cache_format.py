"""The prompt-cache wire format (KVCache.swift:1797-2249): key layout and the restore-time
checks, against the known answers of the reference's KVCacheTests.swift.  Pure host logic,
no device."""
import pytest

from kvhip import prompt_cache as PC


def test_flatten_layout_and_python_compatible_class_name():
    # KVCacheTests.swift:270-287: a KVCacheSimple is stored as "KVCache"; arrays are "i.j",
    # metaState "0.i.j", user metadata "1.key", classes "2.i" (KVCache.swift:1813-1842)
    arrays, meta = PC.flatten([["k0", "v0"], [], ["a", "b", "c", "d", "e", "f"]],
                              [[""], ["0", "32", "256", "0", "0", "modelNative"], ["256", "7", "64", "4"]],
                              [PC.class_name_of("simple"), PC.class_name_of("rotating"), PC.class_name_of("quantized")],
                              {"model": "llama", "a.b": "c"})
    assert arrays == {"0.0": "k0", "0.1": "v0", "2.0": "a", "2.1": "b", "2.2": "c", "2.3": "d", "2.4": "e", "2.5": "f"}
    assert meta["2.0"] == "KVCache" and meta["2.1"] == "RotatingKVCache" and meta["2.2"] == "QuantizedKVCache"
    assert meta["0.0.0"] == "" and meta["0.1.1"] == "32" and meta["0.1.5"] == "modelNative"
    assert [meta[f"0.2.{j}"] for j in range(4)] == ["256", "7", "64", "4"]
    assert meta["1.model"] == "llama" and meta["1.a.b"] == "c"
    info, user, classes = PC.unflatten_metadata(meta)
    assert info == [[""], ["0", "32", "256", "0", "0", "modelNative"], ["256", "7", "64", "4"]]
    assert user == {"model": "llama", "a.b": "c"} and classes == ["KVCache", "RotatingKVCache", "QuantizedKVCache"]
    assert PC.unflatten_arrays(arrays.keys(), 3) == [["0.0", "0.1"], [], ["2.0", "2.1", "2.2", "2.3", "2.4", "2.5"]]


def test_reserved_namespace_and_model_state_are_refused():
    # KVCache.swift:1918-1921, KVCacheTests.swift:318-330
    with pytest.raises(PC.KVCacheError):
        PC.flatten([], [], [], {"__mlx_lm_state_version": "1"})
    # a file carrying model state needs a model runtime (KVCacheTests.swift:259-266)
    with pytest.raises(PC.KVCacheError):
        PC.check_no_model_state(["0.0", "__mlx_lm_state_tensor_0"], {"__mlx_lm_state_count": "1"},
                                ["__mlx_lm_state_v1__:KVCache"])
    # a marker without state is corrupt (KVCacheTests.swift:462-475)
    with pytest.raises(PC.KVCacheError):
        PC.check_no_model_state(["0.0"], {}, ["__mlx_lm_state_v1__:KVCache"])
    PC.check_no_model_state(["0.0", "0.1"], {"note": "x"}, ["KVCache"])


@pytest.mark.parametrize("name,ranks,meta", [
    # KVCacheTests.swift:551-563: incomplete state
    ("KVCacheSimple", [4], [""]),
    ("RotatingKVCache", [4], ["0", "32", "256", "0", "0", "modelNative"]),
    ("QuantizedKVCache", [4, 4, 4], ["256", "0", "64", "4"]),
    # :565-581: invalid metadata
    ("KVCacheSimple", [], ["unexpected"]),
    ("RotatingKVCache", [], ["0", "32", "invalid", "0", "0", "modelNative"]),
    ("RotatingKVCache", [], ["0", "32", "256", "0", "0", "invalid-origin"]),
    ("QuantizedKVCache", [], ["256", "invalid", "64", "4"]),
    # :583-590: invalid rank
    ("KVCacheSimple", [2, 2], [""]),
    # unknown class (KVCache.swift:2147-2149)
    ("SomethingElse", [], [""]),
])
def test_restore_rejections(name, ranks, meta):
    with pytest.raises(PC.KVCacheError):
        PC.plan_restore(name, ranks, meta)


def test_restore_plans():
    assert PC.plan_restore("KVCache", [], [""]) == ("simple", {})
    assert PC.plan_restore("KVCacheSimple", [4, 4], [""]) == ("simple", {})
    # legacy 5-value rotating metadata is accepted (KVCacheTests.swift:592-606)
    assert PC.plan_restore("RotatingKVCache", [4, 4], ["0", "32", "256", "1", "1"]) == ("rotating", {"max_size": 32})
    assert PC.plan_restore("QuantizedKVCache", [4] * 6, ["256", "11", "32", "4"]) == \
        ("quantized", {"group_size": 32, "bits": 4})
    assert PC.plan_restore("QuantizedKVCache", [4] * 4, ["256", "11", "32", "4"])[0] == "quantized"


def test_array_key_corruption():
    # KVCache.swift:2159-2185
    with pytest.raises(PC.KVCacheError):
        PC.unflatten_arrays(["0.0", "1.0"], 1)       # cache index out of range
    with pytest.raises(PC.KVCacheError):
        PC.unflatten_arrays(["0.0", "0.2"], 1)       # non-contiguous
    with pytest.raises(PC.KVCacheError):
        PC.unflatten_arrays(["0"], 1)
