"""Chunk schedule of a prompt on its way into the caches.

`PrefillParameters` (Libraries/MLXLMCommon/PrefillParameters.swift:40-146) decides how many
positions each forward of a long prompt appends -- the `L` of every `update` / `update_attend`
call during prefill.  Host arithmetic only.
"""
from __future__ import annotations

DEFAULT_STEP_SIZE = 512   # PrefillParameters.defaultStepSize (:69)
CHUNKINGS = ("balanced", "remainder", "unchunked")


class PrefillParameters:
    def __init__(self, step_size=None, chunking="balanced", progress=None):
        if chunking not in CHUNKINGS:
            raise ValueError(f"chunking must be one of {CHUNKINGS}")
        self.step_size, self.chunking, self.progress = step_size, chunking, progress

    def resolved_step_size(self, default_step_size=DEFAULT_STEP_SIZE, maximum_step_size=None):
        """`resolvedStepSize` (:73-77): step_size, else the model default, capped, floored at 1."""
        step = self.step_size if self.step_size is not None else default_step_size
        if maximum_step_size is not None:
            step = min(step, maximum_step_size)
        return max(1, step)

    def chunk_length(self, count, default_step_size=DEFAULT_STEP_SIZE, maximum_step_size=None):
        """`chunkLength(forChunking:)` (:86-103): positions per forward, or None (one forward)."""
        step = self.resolved_step_size(default_step_size, maximum_step_size)
        if self.chunking == "unchunked":
            return None
        if self.chunking == "remainder":
            return step
        if count <= step:
            return max(count, 1)
        chunks = (count + step - 1) // step
        return (count + chunks - 1) // chunks

    def for_each_chunk(self, total, body, reserving=1, default_step_size=DEFAULT_STEP_SIZE, maximum_step_size=None):
        """`forEachChunk` (:120-145): calls body(range) per chunk, leaves `reserving` positions for
        the caller's final forward, reports progress, returns the positions processed."""
        length = self.chunk_length(total - reserving, default_step_size, maximum_step_size)
        if length is None:
            return 0
        slack = min(reserving, 1)
        processed = 0
        while total - processed > reserving:
            n = min(length, total - processed - slack)
            body(range(processed, processed + n))
            processed += n
            if self.progress is not None:
                self.progress(processed, total)
        return processed
