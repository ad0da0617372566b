"""CPU restatement of the reference's speculative-round machinery.

TEST INFRASTRUCTURE ONLY: imported by tests/ (and nothing in the product path).

Follows Libraries/MLXLMCommon/KVCacheRound.swift (strategies :99-161, restore
point :163-184, factory :193-218, round :220-252) and the round / timeline part
of `KVCacheStorage` (KVCachePlan.swift:112-399), over the numpy caches of
kv_oracle.py.  It is integer bookkeeping plus array copies, fully specified by
the Swift source, and pinned by the known answers of the reference's own
KVCacheRoundTests.swift (tests/test_oracle_rounds.py).
"""
from __future__ import annotations

import numpy as np

from . import kv_oracle as O


class _WriteThrough:
    # AppendOnlyRoundStrategy, KVCacheRound.swift:99-125
    def __init__(self, slot, live):
        self.slot, self.live, self.start = slot, live, live.offset
        self.presented = live

    def written(self):
        return self.live.offset - self.start

    def commit(self, retaining):
        extra = self.written() - min(max(retaining, 0), self.written())
        if extra > 0:
            self.live.trim(extra)

    def restore_point(self, retaining):
        return None


class _Staged:
    # RotatingRoundStrategy, KVCacheRound.swift:128-161
    def __init__(self, slot, live):
        self.slot, self.live = slot, live
        self.presented = O.RotatingStagedKVCache(live)

    def written(self):
        return self.presented.staged_count

    def commit(self, retaining):
        self.presented.commit(retaining)

    def restore_point(self, retaining):
        if self.live.is_trimmable_after(retaining):
            return None
        snap = self.live.get_state()
        if len(snap) != 2:
            return None
        st = self.presented
        replay = None if st.staged_keys is None else (np.array(st.staged_keys), np.array(st.staged_values))
        return dict(state=[np.array(a) for a in snap], meta=list(self.live.get_meta_state()), replay=replay)


def _restore(point, leaf, retaining):
    # RotatingRestorePoint.restore, KVCacheRound.swift:171-183
    leaf.set_state([np.array(a) for a in point["state"]])
    leaf.set_meta_state(list(point["meta"]))
    if retaining > 0 and point["replay"] is not None:
        leaf.update(point["replay"][0][:, :, :retaining], point["replay"][1][:, :, :retaining])


class Storage:
    """`KVCacheStorage` rounds and timeline (KVCachePlan.swift:112-399)."""

    def __init__(self, caches, processed=None):
        self.cache = list(caches)
        self.processed = min([c.offset for c in self.cache], default=0) if processed is None else processed
        self.open = None
        self.last = None

    def commit_processed_tokens(self, n):
        self.processed += n
        self.last = None

    def replace(self, caches):
        self.cache = list(caches)
        self.last = None

    def trim(self, n):
        assert self.open is None
        t = O.trim_prompt_cache(self.cache, n)
        self.processed -= t
        self.last = None
        return t

    def begin_round(self, width):
        assert self.open is None
        strategies = []
        for slot, leaf in enumerate(self.cache):
            if isinstance(leaf, O.RotatingKVCache):
                strategies.append((slot, "staged"))
            elif hasattr(leaf, "is_trimmable_after") and leaf.is_trimmable_after(width):
                strategies.append((slot, "through"))
            else:
                return None
        self.last = None
        self.open = [(_Staged if k == "staged" else _WriteThrough)(s, self.cache[s]) for s, k in strategies]
        return self.open

    def commit(self, round_, retaining):
        assert self.open is round_
        written = round_[0].written() if round_ else 0
        assert all(s.written() == written for s in round_)
        assert 0 <= retaining <= written
        records = []
        for s in round_:
            records.append((s.slot, s.restore_point(retaining)))
            s.commit(retaining)
        self.processed += retaining
        self.open = None
        self.last = (retaining, records) if any(p is not None for _, p in records) else None
        return retaining, written - retaining

    def rewind_last_round(self, count):
        assert self.open is None
        if count <= 0:
            return 0
        if self.last is None:
            return self.trim(count)
        committed, records = self.last
        rewound = min(count, committed)
        if rewound <= 0:
            return 0
        for slot, point in records:
            if slot >= len(self.cache):
                return self.trim(count)
            leaf = self.cache[slot]
            if (point is not None and not isinstance(leaf, O.RotatingKVCache)) or \
               (point is None and not leaf.is_trimmable):
                return self.trim(count)
        for slot, point in records:
            leaf = self.cache[slot]
            if point is not None:
                _restore(point, leaf, committed - rewound)
            else:
                assert leaf.trim(rewound) == rewound
        self.processed -= rewound
        self.last = None
        return rewound

    def copy(self):
        assert self.open is None
        return Storage([c.copy() for c in self.cache], self.processed)

    def aligned(self):
        return all(c.offset == self.processed for c in self.cache)
