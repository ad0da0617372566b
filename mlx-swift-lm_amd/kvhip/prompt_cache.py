"""Prompt-cache files in the reference's wire format.

`savePromptCache` / `loadPromptCache` (Libraries/MLXLMCommon/KVCache.swift:1797-2249)
write one safetensors file: arrays keyed "i.j" (cache i, state array j) and string
metadata flattened as "0.i.j" (cache i's metaState entry j), "1.key" (user metadata)
and "2.i" (cache i's class name; `KVCacheSimple` is stored under the Python-compatible
name "KVCache", KVCache.swift:1739-1751).  A device cache exports `state` / `meta_state`
through the C ABI in exactly those layouts, so files written here load in the reference
(and in mlx-lm) and the other way round.

Files that carry model state ("__mlx_lm_state_" entries, KVCache.swift:1894-2020) belong
to a model runtime; this library has no model state type and refuses them, the way the
reference's tuple-returning `loadPromptCache` does.
"""
from __future__ import annotations

import re

STATE_METADATA_PREFIX = "__mlx_lm_state_"          # KVCache.swift:2011-2018
STATE_TENSOR_PREFIX = "__mlx_lm_state_tensor_"
STATE_CLASS_PREFIX = "__mlx_lm_state_v1__:"

CAPACITY_ORIGINS = ("modelNative", "requested")


class KVCacheError(ValueError):
    """`KVCacheError` (KVCache.swift:1730-1734): a recoverable load / conversion failure."""


# ---------------------------------------------------------------------------------
# pure format logic (no device, no file): shared by save, load and the CPU tests
# ---------------------------------------------------------------------------------

def class_name_of(kind):
    """`cacheClassName` (KVCache.swift:1739-1751) for the three kinds of this library."""
    return {"simple": "KVCache", "rotating": "RotatingKVCache", "quantized": "QuantizedKVCache"}[kind]


def flatten(states, infos, class_names, user_metadata):
    """-> (arrays dict "i.j", metadata dict) as `savePromptCache` lays them out (:1813-1842)."""
    for key in user_metadata:
        if key.startswith(STATE_METADATA_PREFIX):
            raise KVCacheError("User metadata uses the reserved prompt cache state namespace")
    arrays, meta = {}, {}
    for i, state in enumerate(states):
        for j, a in enumerate(state):
            arrays[f"{i}.{j}"] = a
    for i, info in enumerate(infos):
        for j, value in enumerate(info):
            meta[f"0.{i}.{j}"] = value
    for key, value in user_metadata.items():
        meta[f"1.{key}"] = value
    for i, name in enumerate(class_names):
        meta[f"2.{i}"] = name
    return arrays, meta


def unflatten_metadata(flat):
    """`unflattenMetadata` (KVCache.swift:2192-2232): [cache_info, user_metadata, cache_classes]."""
    cache_info, user, classes = [], {}, []
    for key, value in flat.items():
        parts = key.split(".")
        if len(parts) >= 3 and parts[0] == "0":
            if parts[1].isdigit() and parts[2].isdigit():
                i, j = int(parts[1]), int(parts[2])
                while len(cache_info) <= i:
                    cache_info.append([])
                while len(cache_info[i]) <= j:
                    cache_info[i].append("")
                cache_info[i][j] = value
        elif len(parts) >= 2 and parts[0] == "1":
            user[".".join(parts[1:])] = value
        elif len(parts) >= 2 and parts[0] == "2":
            if parts[1].isdigit():
                i = int(parts[1])
                while len(classes) <= i:
                    classes.append("")
                classes[i] = value
    return cache_info, user, classes


def unflatten_arrays(keys, cache_count):
    """`unflattenArrays` (KVCache.swift:2151-2189) on the keys alone: per cache the ordered
    list of its array keys."""
    by_cache = {}
    for key in keys:
        m = re.fullmatch(r"(\d+)\.(\d+)", key)
        if not m or not (0 <= int(m.group(1)) < cache_count):
            raise KVCacheError(f"Corrupt prompt cache: invalid array key '{key}'.")
        by_cache.setdefault(int(m.group(1)), {})[int(m.group(2))] = key
    out = []
    for i in range(cache_count):
        entries = by_cache.get(i, {})
        ordered = []
        for j in range(len(entries)):
            if j not in entries:
                raise KVCacheError(f"Corrupt prompt cache: cache {i} has non-contiguous array indices.")
            ordered.append(entries[j])
        out.append(ordered)
    return out


def _integers(values, class_name):
    out = []
    for v in values:
        if not re.fullmatch(r"[+-]?\d+", v):
            raise KVCacheError(f"Corrupt prompt cache: {class_name} metadata must contain integers.")
        out.append(int(v))
    return out


def plan_restore(class_name, state_ranks, meta_state):
    """The checks of `restoreCacheFromMetaState` (KVCache.swift:2026-2150) for the classes of
    this library.  -> (kind, constructor arguments)."""
    def validate(name, state_counts, meta_counts):
        if len(state_ranks) not in state_counts or len(meta_state) not in meta_counts or \
                any(rank != 4 for rank in state_ranks):
            raise KVCacheError(f"Corrupt prompt cache: invalid {name} state or metadata shape.")

    if class_name in ("KVCache", "KVCacheSimple"):
        validate("KVCacheSimple", (0, 2), (1,))
        if meta_state != [""]:
            raise KVCacheError("Corrupt prompt cache: KVCacheSimple metadata must contain its single "
                               "empty placeholder.")
        return "simple", {}
    if class_name == "RotatingKVCache":
        validate(class_name, (0, 2), (5, 6))
        values = _integers(meta_state[:5], class_name)
        if len(meta_state) == 6 and meta_state[5] not in CAPACITY_ORIGINS:
            raise KVCacheError(f"Corrupt prompt cache: invalid RotatingKVCache capacity origin '{meta_state[5]}'.")
        return "rotating", {"max_size": values[1]}
    if class_name == "QuantizedKVCache":
        validate(class_name, (0, 4, 6), (4,))
        values = _integers(meta_state, class_name)
        return "quantized", {"group_size": values[2], "bits": values[3]}
    raise KVCacheError(f"Unknown cache class: {class_name}")


def check_no_model_state(array_keys, user_metadata, class_names):
    """A file with model state needs a model runtime (KVCache.swift:1864-1876, :1991-2009)."""
    has_state = any(k.startswith(STATE_METADATA_PREFIX) for k in user_metadata) or \
        any(k.startswith(STATE_TENSOR_PREFIX) for k in array_keys)
    if has_state:
        raise KVCacheError("Prompt cache contains model state; it needs the model runtime that wrote it")
    if any(name.startswith(STATE_CLASS_PREFIX) for name in class_names):
        raise KVCacheError("Prompt cache compatibility marker has no model state")


# ---------------------------------------------------------------------------------
# device caches <-> files
# ---------------------------------------------------------------------------------

def _kind_of(cache):
    from . import cache as C
    if isinstance(cache, C.RotatingKVCache):
        return "rotating"
    if isinstance(cache, C.QuantizedKVCache):
        return "quantized"
    if isinstance(cache, C.KVCacheSimple):
        return "simple"
    raise KVCacheError(f"cannot serialize a {type(cache).__name__}")


def save_prompt_cache(path, caches, metadata=None):
    """`savePromptCache(url:cache:metadata:)` (KVCache.swift:1797-1845)."""
    import torch
    from safetensors.torch import save_file

    states, infos, names = [], [], []
    for c in caches:
        arrays = []
        for a in c.state:
            # packed codes travel as uint32, the dtype MLX gives them
            arrays.append((a.view(torch.uint32) if a.dtype == torch.int32 else a).contiguous().cpu())
        states.append(arrays)
        infos.append(list(c.meta_state))
        names.append(class_name_of(_kind_of(c)))
    arrays, meta = flatten(states, infos, names, dict(metadata or {}))
    save_file(arrays, str(path), metadata=meta)


def load_prompt_cache(path):
    """`loadPromptCache(url:)` (KVCache.swift:1859-1912): (caches, user metadata)."""
    import torch
    from safetensors import safe_open

    from . import cache as C

    with safe_open(str(path), "pt") as f:
        flat_meta = f.metadata() or {}
        keys = list(f.keys())
        cache_info, user, classes = unflatten_metadata(flat_meta)
        check_no_model_state(keys, user, classes)
        if len(cache_info) != len(classes):
            raise KVCacheError("Mismatch in cache counts")
        per_cache = unflatten_arrays(keys, len(classes))
        caches = []
        for i, name in enumerate(classes):
            tensors = [f.get_tensor(k) for k in per_cache[i]]
            kind, args = plan_restore(name, [t.dim() for t in tensors], cache_info[i])
            if kind == "simple":
                c = C.KVCacheSimple()
            elif kind == "rotating":
                c = C.RotatingKVCache(args["max_size"])
            else:
                c = C.QuantizedKVCache(args["group_size"], args["bits"])
            if tensors:
                c.state = [(t.view(torch.int32) if t.dtype == torch.uint32 else t).cuda() for t in tensors]
            if kind != "simple":
                c.meta_state = cache_info[i]
            caches.append(c)
    return caches, user
