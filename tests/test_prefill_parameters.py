"""`kvhip.prefill.PrefillParameters` against the known answers of the reference's
Tests/MLXLMTests/PrefillParametersTests.swift (chunk-length arithmetic :16-65, schedules :83-112)."""
import importlib.util
import os

import pytest

_spec = importlib.util.spec_from_file_location(
    "kvhip_prefill", os.path.join(os.path.dirname(__file__), "..", "mlx-swift-lm_amd", "kvhip", "prefill.py"))
P = importlib.util.module_from_spec(_spec)
_spec.loader.exec_module(P)


def test_balanced_arithmetic():
    prefill = P.PrefillParameters(None, "balanced")
    for count, step in [(31884, 1024), (5000, 512), (1025, 1024), (7, 3), (100, 100)]:
        chunk = prefill.chunk_length(count, default_step_size=step)
        assert chunk <= step
        minimal = (count + step - 1) // step
        assert (count + chunk - 1) // chunk == minimal
        last = count - (minimal - 1) * chunk
        assert chunk - minimal < last <= chunk


def test_balanced_degenerates():
    prefill = P.PrefillParameters(chunking="balanced")
    assert prefill.chunk_length(24, default_step_size=128) == 24
    assert prefill.chunk_length(512, default_step_size=512) == 512
    assert prefill.chunk_length(0, default_step_size=512) == 1
    assert P.PrefillParameters(step_size=0).chunk_length(10, default_step_size=512) == 1


def test_step_resolution():
    assert P.PrefillParameters(8, "remainder").chunk_length(100, default_step_size=512) == 8
    assert P.PrefillParameters(512, "remainder").chunk_length(100, default_step_size=128, maximum_step_size=64) == 64
    assert P.PrefillParameters(chunking="remainder").chunk_length(100, default_step_size=128, maximum_step_size=64) == 64


def test_unchunked_is_none():
    prefill = P.PrefillParameters(chunking="unchunked")
    assert prefill.chunk_length(5) is None and prefill.chunk_length(31884) is None


def schedule(total, prefill, reserving=1):
    chunks = []
    processed = prefill.for_each_chunk(total, chunks.append, reserving=reserving)
    return chunks, total - processed


def test_schedule_pin_31885_tokens_at_1024():
    chunks, tail = schedule(31885, P.PrefillParameters(1024, "balanced"))
    assert [len(c) for c in chunks] == [997] * 31 + [977]
    assert chunks[0].start == 0 and chunks[-1].stop == 31884 and tail == 1
    chunks, tail = schedule(31885, P.PrefillParameters(1024, "remainder"), reserving=1024)
    assert [len(c) for c in chunks] == [1024] * 31 and tail == 141


def test_schedule_short_prompt_and_progress():
    events = []
    chunks, tail = schedule(300, P.PrefillParameters(512, "balanced", progress=lambda p, t: events.append((p, t))))
    assert [len(c) for c in chunks] == [299] and tail == 1 and events == [(299, 300)]
    chunks, tail = schedule(300, P.PrefillParameters(512, "unchunked"))
    assert chunks == [] and tail == 300
    with pytest.raises(ValueError):
        P.PrefillParameters(chunking="sometimes")
