"""The decode loop of `TokenIterator` (Evaluate.swift:905-952) over a stack of layer caches, through
the C ABI: per step every layer rotates its queries and keys at the cache's `ropeOffset`, writes the
cache and attends (Llama.swift:58-70, AttentionUtils.swift:37-95); then `commitProcessedTokens`, then the
dynamic conversion of `kvCachePlan.apply` (`maybeAffineQuantizeKVCache`, KVCache.swift:2500-2520); the host
waits for the previous step's output only (`asyncEval` of step t, `item()` of step t - 1).

Checked: every layer's final state against the oracle (bit-exact: codes, scale / bias pairs, rows, ring
order, metaState), every step's last-layer output within max-abs 1e-2 / mean-abs 1e-3, and that the
library calls of a whole step -- one that appends device pages and one that converts caches included --
only enqueue: with the stream held busy by a long kernel they return while it is still running.
"""
import time

import numpy as np
import pytest
import torch

import kvhip
from oracle import kv_oracle as O
from oracle import rope as ORope
from tests.util import bits_equal, dev, err_stats, np32

pytestmark = pytest.mark.gpu

B, HQ, HKV, D = 2, 8, 2, 64
DT, NAME = torch.float16, "float16"
SCALE = D ** -0.5
WINDOW = 128
LAYERS = ["simple", "ring", "simple", "quant8", "simple", "ring_keep", "quant4", "simple"] * 2   # 16 layers
PROMPT, STEPS = 200, 90          # offsets run from 200 to 290: every unbounded cache crosses the 256-row page
COMPRESSION_START = 230          # KVCachePlan's affine scheme: simple caches convert once offset > 230
BITS, GS = 4, 64


def make_layers():
    dev_caches, ora_caches = [], []
    for kind in LAYERS:
        if kind == "simple":
            dev_caches.append(kvhip.KVCacheSimple())
            ora_caches.append(O.KVCacheSimple(NAME))
        elif kind == "ring":
            dev_caches.append(kvhip.RotatingKVCache(WINDOW))
            ora_caches.append(O.RotatingKVCache(WINDOW, dtype=NAME))
        elif kind == "ring_keep":
            dev_caches.append(kvhip.RotatingKVCache(WINDOW, keep=4))
            ora_caches.append(O.RotatingKVCache(WINDOW, keep=4, dtype=NAME))
        else:
            bits = 8 if kind == "quant8" else 4
            dev_caches.append(kvhip.QuantizedKVCache(64, bits))
            ora_caches.append(O.QuantizedKVCache(64, bits, NAME))
    return dev_caches, ora_caches


def oracle_maybe_quantize(caches):
    for i, c in enumerate(caches):
        if type(c) is O.KVCacheSimple and c.offset > COMPRESSION_START:
            caches[i] = c.to_quantized(GS, BITS)


def oracle_mask(cache, n):
    if isinstance(cache, O.RotatingKVCache):
        return cache.make_mask(n, None, False)
    return O.base_make_mask(cache.offset, n, None, False)


def oracle_layer(cache, q_rot, k_rot, v):
    """`attentionWithCacheUpdate` on rows that already carry their rotary positions."""
    return O.attention_with_cache_update(q_rot, k_rot, v, cache, SCALE, oracle_mask(cache, q_rot.shape[2]), NAME)


def device_layer(rope, cache, qd, kd, vd):
    """What an attention layer does (Llama.swift:58-70): rotate queries and keys at the cache's ropeOffset,
    write the cache (the key rotation runs inside the append kernel), attend.  Also returns the rotated
    queries and, from one more launch that only the checker needs, the rotated keys: the oracle is fed the
    very rows the cache received (the rotation itself is checked in tests/test_gpu_rope.py, where the fused
    append is bit-identical to rotate-then-append)."""
    mask = kvhip.create_attention_mask(qd.shape[2], cache)
    q_rot = kvhip.apply_rotary_position(rope, qd, cache)
    k_rot = kvhip.apply_rotary_position(rope, kd, cache)
    cache.update_rope(rope, kd, vd)
    return cache.attend(q_rot, SCALE, mask), q_rot, k_rot


def check_states(dev_caches, ora_caches):
    for li, (c, o) in enumerate(zip(dev_caches, ora_caches)):
        assert c.offset == o.offset, (li, c.offset, o.offset)
        assert c.meta_state == o.get_meta_state(), li
        quant = isinstance(o, O.QuantizedKVCache)
        assert isinstance(c, kvhip.QuantizedKVCache) == quant, (li, type(c))
        for i, (a, b) in enumerate(zip(c.state, o.get_state())):
            assert tuple(a.shape) == tuple(b.shape), (li, i)
            if quant and i % 3 == 0:
                assert np.array_equal(np32(a), b), (li, i)
            else:
                assert bits_equal(a, b, DT), (li, i)


def test_decode_loop_matches_the_oracle_and_only_enqueues():
    rng = np.random.default_rng(41)
    nl = len(LAYERS)
    rope = kvhip.RoPE(D)
    dev_caches, ora_caches = make_layers()
    storage = kvhip.KVCacheStorage(dev_caches)

    def draw(shape):
        a = O.round_to(rng.standard_normal(shape).astype(np.float32), NAME)
        return a, dev(a, DT)

    def forward(n):
        """One model forward over all layers, enqueued only.  A layer's queries take a tenth of the output of
        the layer below, which makes the launches of a step a dependent chain."""
        rec, prev_d = [], None
        for li in range(nl):
            (_, qd), (_, kd), (v, vd) = draw((B, HQ, n, D)), draw((B, HKV, n, D)), draw((B, HKV, n, D))
            if prev_d is not None:
                qd = (qd.float() + 0.1 * prev_d.float()).to(DT)
            prev_d, q_rot, k_rot = device_layer(rope, storage.cache[li], qd, kd, vd)
            rec.append((q_rot, k_rot, v, prev_d))
        return rec

    def oracle_step(rec_host, label):
        for li, (q_rot, k_rot, v, out) in enumerate(rec_host):
            ref = oracle_layer(ora_caches[li], q_rot, k_rot, v)
            mx, mean = err_stats(out, ref)
            assert mx <= 1e-2 and mean <= 1e-3, (label, li, mx, mean)

    # ---- prompt: one chunk through every layer (Evaluate.swift:845-880 prepares the cache this way) ----
    rec = forward(PROMPT)
    storage.commit_processed_tokens(PROMPT)
    oracle_step([(np32(q), np32(k), v, np32(o)) for q, k, v, o in rec], "prompt")
    check_states(storage.cache, ora_caches)

    # ---- decode: step t is enqueued in full before the host waits for step t - 1 ------------------------
    copy_stream = torch.cuda.Stream()
    pending = None            # (event behind step t - 1, what it recorded, t - 1)
    grew = converted = 0
    held_steps = []

    def settle(pending):
        """Wait for that step only -- its rows are copied out on another stream behind its event -- and run
        the oracle's step on them."""
        ev, rec, step = pending
        with torch.cuda.stream(copy_stream):
            copy_stream.wait_event(ev)
            host = [(q.to("cpu", non_blocking=True), k.to("cpu", non_blocking=True), v, o.to("cpu", non_blocking=True))
                    for q, k, v, o in rec]
            got = torch.cuda.Event()
            got.record(copy_stream)
        got.synchronize()
        oracle_step([(q.float().numpy(), k.float().numpy(), v, o.float().numpy()) for q, k, v, o in host], step)
        oracle_maybe_quantize(ora_caches)

    for t in range(STEPS):
        rows_before = [c.device_rows for c in storage.cache]
        kinds_before = [type(c) for c in storage.cache]
        # a step that will grow pages (offset 256) or convert caches (offset 230 -> 231): keep the stream busy with
        # a long kernel first, so that a call which waited for the device would show
        hold = (PROMPT + t) in (COMPRESSION_START, 256)
        if hold:
            torch.cuda._sleep(int(4e7))       # tens of milliseconds of device time in front of this step
        h0 = time.perf_counter()
        rec = forward(1)
        storage.commit_processed_tokens(1)
        kvhip.maybe_affine_quantize_kv_cache(storage.cache, BITS, GS, COMPRESSION_START)
        host_s = time.perf_counter() - h0
        if hold:
            held_steps.append((PROMPT + t, host_s, not torch.cuda.current_stream().query()))
        done = torch.cuda.Event()
        done.record()
        grew += sum(c.device_rows != r for c, r in zip(storage.cache, rows_before))
        converted += sum(type(c) is not k for c, k in zip(storage.cache, kinds_before))
        if pending is not None:
            settle(pending)
        pending = (done, rec, t)
    settle(pending)
    torch.cuda.synchronize()
    assert storage.processed_token_count == PROMPT + STEPS
    # what the loop went through on the way
    assert converted == LAYERS.count("simple") and grew >= LAYERS.count("simple") + 4, (converted, grew)
    check_states(storage.cache, ora_caches)
    # the held steps returned while the long kernel in front of them was still running
    assert [o for o, _, _ in held_steps] == [COMPRESSION_START, 256]
    for offset, host_s, busy in held_steps:
        assert busy, f"the step at offset {offset} waited for the device ({host_s * 1e3:.1f} ms on the host)"
