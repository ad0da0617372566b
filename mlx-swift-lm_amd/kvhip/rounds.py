"""Speculative rounds over device caches: host-side mirror of the reference's
round machinery.

`RotatingStagedKVCache` follows Libraries/MLXLMCommon/RotatingStagedKVCache.swift:12-132,
the strategies and restore point KVCacheRound.swift:17-252, and `KVCacheStorage`
KVCachePlan.swift:112-399 (the round / timeline part).  All of it is integer
bookkeeping on the host; the rows themselves stay on the device: a staged round on
a ring writes its rows into spare slots of the ring's page store and attention
reads the trailing window plus the staged rows in place (no concatenation), and a
commit appends the kept prefix through the ring's normal write path.
"""
from __future__ import annotations

import torch

from . import _lib as L
from .cache import RotatingKVCache, _ptr, _stream, trim_prompt_cache


class RotatingStagedKVCache:
    """A `RotatingKVCache` presented with uncommitted rows appended
    (RotatingStagedKVCache.swift:12-132).  Shares the live cache's device handle."""

    def __init__(self, live: RotatingKVCache):
        self.live = live
        L.check(live._lib.kvhip_cache_stage_begin(live._h))
        self._open = True

    # -- protocol surface ----------------------------------------------------
    @property
    def staged_count(self):
        return self.live._lib.kvhip_cache_stage_count(self.live._h) if self._open else 0

    @property
    def staged_arrays(self):
        """`stagedArrays` (:27-30): the staged rows, valid until commit."""
        n = self.staged_count
        if n == 0:
            return None
        B, H, Dk, Dv, dt = self.live._shape
        k = torch.empty((B, H, n, Dk), dtype=dt, device="cuda")
        v = torch.empty((B, H, n, Dv), dtype=dt, device="cuda")
        L.check(self.live._lib.kvhip_cache_stage_fetch(self.live._h, _ptr(k), _ptr(v), _stream()))
        return k, v

    @property
    def offset(self):
        return self.live.offset + self.staged_count

    @property
    def rope_offset(self):
        return self.offset

    @property
    def max_size(self):
        return self.live.max_size

    @property
    def presented_length(self):
        return self.live.presented_length

    def update_rope(self, rope, keys, values, batch_offsets=None):
        self._require_open()
        return self.live.update_rope(rope, keys, values, batch_offsets)

    def update(self, keys, values, fetch=True):
        """Stages the rows; returns trailing window ++ staged (:41-47, :78-91)."""
        self._require_open()
        return self.live.update(keys, values, fetch=fetch)

    def attend(self, queries, scale, mask=None):
        return self.live.attend(queries, scale, mask)

    def update_attend(self, queries, keys, values, scale, mask=None):
        self._require_open()
        return self.live.update_attend(queries, keys, values, scale, mask)

    def make_mask(self, n, window_size=None, return_array=False):
        """The live cache's own mask (:49-58)."""
        return self.live.make_mask(n, window_size, return_array)

    def commit(self, retaining):
        """`commit(retaining:)` (:62-76)."""
        if not self._open:
            return
        self._open = False
        L.check(self.live._lib.kvhip_cache_stage_commit(self.live._h, int(retaining), _stream()))

    # -- round-scoped: not serializable, not rewindable, not copyable (:93-125) --------
    @property
    def state(self):
        return self.live.state

    @state.setter
    def state(self, arrays):
        raise RuntimeError("RotatingStagedKVCache is round-scoped and cannot be restored from state "
                           f"({len(arrays)} arrays)")

    @property
    def meta_state(self):
        return self.live.meta_state

    @meta_state.setter
    def meta_state(self, values):
        raise RuntimeError("RotatingStagedKVCache is round-scoped and cannot be restored from metaState "
                           f"({len(values)} values)")

    is_trimmable = False

    def is_trimmable_after(self, positions):
        return False

    def trim(self, n):
        return 0

    def copy(self):
        raise RuntimeError("RotatingStagedKVCache is round-scoped and cannot be copied")

    def _require_open(self):
        if not self._open:
            raise RuntimeError("the staged round of this cache has been committed")


# ---------------------------------------------------------------------------------
# strategies (KVCacheRound.swift)
# ---------------------------------------------------------------------------------

class AppendOnlyRoundStrategy:
    """Written through, then clamped back over the rejected rows (KVCacheRound.swift:99-125)."""

    def __init__(self, slot, live):
        self.slot, self.live = slot, live
        self._start = live.offset

    @property
    def presented(self):
        return self.live

    @property
    def written_positions(self):
        return self.live.offset - self._start

    @property
    def live_offset(self):
        return self.live.offset

    @property
    def attention_bound(self):
        return self.live.max_size

    def commit(self, retaining):
        written = self.written_positions
        keep = min(max(retaining, 0), written)
        if written > keep:
            self.live.trim(written - keep)

    def make_restore_point(self, retaining):
        return None


class RotatingRestorePoint:
    """Puts a ring back and replays the accepted rows (KVCacheRound.swift:163-184)."""

    def __init__(self, state, meta_state, replay):
        self.state, self.meta_state, self.replay = state, meta_state, replay

    def can_restore(self, leaf):
        return isinstance(leaf, RotatingKVCache)

    def restore(self, leaf, retaining):
        if not isinstance(leaf, RotatingKVCache):
            return False
        leaf.state = self.state
        leaf.meta_state = self.meta_state
        if retaining > 0 and self.replay is not None:
            leaf.update(self.replay[0][:, :, :retaining], self.replay[1][:, :, :retaining], fetch=False)
        return True


class RotatingRoundStrategy:
    """Staged beside the ring, which stays untouched until commit (KVCacheRound.swift:128-161)."""

    def __init__(self, slot, live: RotatingKVCache):
        self.slot, self.live = slot, live
        self.staged = RotatingStagedKVCache(live)

    @property
    def presented(self):
        return self.staged

    @property
    def written_positions(self):
        return self.staged.staged_count

    @property
    def live_offset(self):
        return self.live.offset

    @property
    def attention_bound(self):
        return self.live.max_size

    def commit(self, retaining):
        self.staged.commit(retaining)

    def make_restore_point(self, retaining):
        # below the window a trim is exact bookkeeping: no snapshot (KVCacheRound.swift:146-150)
        if self.live.is_trimmable_after(retaining):
            return None
        snapshot = self.live.state
        if len(snapshot) != 2:
            return None
        return RotatingRestorePoint(snapshot, self.live.meta_state, self.staged.staged_arrays)


def _emitted_length(strategy):
    bound = strategy.attention_bound
    return strategy.live_offset if bound is None else min(strategy.live_offset, bound)


def make_round_strategy(leaf, slot, maximum_positions):
    """`KVCacheRoundStrategyFactory.make` (KVCacheRound.swift:193-218) for the cache kinds of
    this library; anything else is judged by `is_trimmable_after` when it has one."""
    if isinstance(leaf, RotatingKVCache):
        return RotatingRoundStrategy(slot, leaf)
    probe = getattr(leaf, "is_trimmable_after", None)
    ok = probe(maximum_positions) if probe is not None else bool(getattr(leaf, "is_trimmable", False))
    if not ok or not hasattr(leaf, "trim") or not hasattr(leaf, "offset"):
        return None
    return AppendOnlyRoundStrategy(slot, leaf)


class KVCacheRound:
    """An open staged round (KVCacheRound.swift:220-247)."""

    def __init__(self, strategies, maximum_positions):
        self.strategies = strategies
        self.caches = [s.presented for s in strategies]
        self.maximum_positions = maximum_positions

    @property
    def written_positions(self):
        if not self.strategies:
            return 0
        written = [s.written_positions for s in self.strategies]
        assert all(w == written[0] for w in written), f"leaves disagree on how much this round wrote: {written}"
        return written[0]


class KVCacheRoundCommit:
    """`KVCacheRoundCommit` (KVCacheRound.swift:250-252)."""

    def __init__(self, committed, discarded, emitted_lengths):
        self.committed_positions = committed
        self.discarded_positions = discarded
        self.emitted_lengths = emitted_lengths


class KVCacheStorage:
    """The round / timeline part of `KVCacheStorage` (KVCachePlan.swift:112-399)."""

    def __init__(self, cache, processed_token_count=None):
        self._cache = list(cache)
        self._open_round = None
        self._last_round = None  # (committed positions, [(slot, restore point or None)])
        if processed_token_count is None:
            def leaves(entries):
                for e in entries:
                    if isinstance(e, (list, tuple)):
                        yield from leaves(e)
                    else:
                        yield e
            offsets = [c.offset for c in leaves(self._cache)]
            processed_token_count = min(offsets) if offsets else 0
        self.processed_token_count = processed_token_count

    @property
    def cache(self):
        return self._cache

    def replace(self, cache):
        assert not self.round_is_open, "the realized cache was replaced while a staged round was open"
        self._cache = list(cache)
        self._last_round = None

    @property
    def round_is_open(self):
        return self._open_round is not None

    def commit_processed_tokens(self, count):
        assert count >= 0, "Processed token count cannot move backwards"
        self.processed_token_count += count
        self._last_round = None

    def trim(self, count):
        assert count >= 0, "Trim count cannot be negative"
        assert not self.round_is_open, "cannot trim while a staged round is open"
        trimmed = trim_prompt_cache(self._cache, count)
        assert trimmed <= self.processed_token_count, "Cache trimmed beyond its processed-token timeline"
        self.processed_token_count -= trimmed
        self._last_round = None
        return trimmed

    def begin_round(self, maximum_positions):
        """`beginRound(maximumPositions:)` (KVCachePlan.swift:219-244): None when a leaf cannot
        take part, with nothing touched."""
        assert not self.round_is_open, "a staged round is already open on this storage"
        # classify every leaf before constructing anything: a staged wrapper opens device state
        kinds = []
        for leaf in self._cache:
            if isinstance(leaf, (list, tuple)):
                return None  # nested topologies are refused
            if isinstance(leaf, RotatingKVCache):
                kinds.append("rotating")
                continue
            probe = getattr(leaf, "is_trimmable_after", None)
            ok = probe(maximum_positions) if probe is not None else bool(getattr(leaf, "is_trimmable", False))
            if not ok or not hasattr(leaf, "trim") or not hasattr(leaf, "offset"):
                return None
            kinds.append("append")
        strategies = [make_round_strategy(leaf, slot, maximum_positions) for slot, leaf in enumerate(self._cache)]
        self._last_round = None
        self._open_round = KVCacheRound(strategies, maximum_positions)
        return self._open_round

    def commit(self, round_, retaining):
        """`commit(_:retaining:)` (KVCachePlan.swift:253-294)."""
        assert self._open_round is round_, "committing a round that is not open on this storage"
        written = round_.written_positions
        assert 0 <= retaining <= written, f"cannot retain {retaining} of {written} written positions"
        rewinds = []
        for strategy in round_.strategies:
            rewinds.append((strategy.slot, strategy.make_restore_point(retaining)))
            strategy.commit(retaining)
        self.processed_token_count += retaining
        self._open_round = None
        self._last_round = (retaining, rewinds) if any(p is not None for _, p in rewinds) else None
        return KVCacheRoundCommit(retaining, written - retaining, [_emitted_length(s) for s in round_.strategies])

    def rollback(self, round_):
        return self.commit(round_, 0)

    def rewind_last_round(self, count):
        """`rewindLastRound(_:)` (KVCachePlan.swift:309-358)."""
        assert count >= 0, "Rewind count cannot be negative"
        assert not self.round_is_open, "cannot rewind while a staged round is open"
        if count <= 0:
            return 0
        if self._last_round is None:
            return self.trim(count)
        committed, records = self._last_round
        rewound = min(count, committed)
        if rewound <= 0:
            return 0
        resolved = []
        for slot, point in records:
            if not (0 <= slot < len(self._cache)):
                return self.trim(count)
            leaf = self._cache[slot]
            ok = point.can_restore(leaf) if point is not None else bool(leaf.is_trimmable)
            if not ok:
                return self.trim(count)
            resolved.append((slot, point, leaf))
        for slot, point, leaf in resolved:
            if point is not None:
                point.restore(leaf, committed - rewound)
            else:
                trimmed = leaf.trim(rewound)
                assert trimmed == rewound, f"entry {slot} took back {trimmed} of {rewound} positions"
        self.processed_token_count -= rewound
        self._last_round = None
        return rewound

    def emitted_length(self, index):
        if not (0 <= index < len(self._cache)):
            return self.processed_token_count
        bound = self._cache[index].max_size
        return self.processed_token_count if bound is None else min(self.processed_token_count, bound)

    def copy(self):
        assert not self.round_is_open, "cannot snapshot while a staged round is open"
        return KVCacheStorage([c.copy() for c in self._cache], self.processed_token_count)

    @property
    def native_attention_offsets_are_aligned(self):
        return all(c.offset == self.processed_token_count for c in self._cache)
