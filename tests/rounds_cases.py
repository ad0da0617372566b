"""Known-answer cases for speculative rounds, restated from the reference's own
KVCacheRoundTests.swift and written once against a small backend interface, so the
CPU oracle (tests/test_oracle_rounds.py) and the device path through the C ABI
(tests/test_gpu_rounds.py) are held to the same integers.

Rows encode their own sequence position (keys +p, values -p), as in
KVCacheRoundTests.swift:13-30: any reordering, duplication or K/V mix-up changes
the numbers.
"""
import numpy as np


class Backend:
    """What a case needs from an implementation."""
    def rotating(self, max_size, keep=0): raise NotImplementedError
    def simple(self): raise NotImplementedError
    def storage(self, caches): raise NotImplementedError
    def kv(self, lo, hi): raise NotImplementedError            # positioned (keys, values)
    def update(self, cache, k, v): raise NotImplementedError   # -> presented (keys, values)
    def positions(self, keys): raise NotImplementedError       # [B,H,S,D] -> [int]
    def view(self, cache, tail): raise NotImplementedError     # logicalView or None
    def meta(self, cache): raise NotImplementedError
    def state(self, cache): raise NotImplementedError          # list of numpy arrays
    def is_staged(self, cache): raise NotImplementedError
    def staged_count(self, cache): raise NotImplementedError
    # storage
    def begin(self, st, width): raise NotImplementedError
    def caches_of(self, rnd): raise NotImplementedError
    def commit(self, st, rnd, n): raise NotImplementedError
    def rewind(self, st, n): raise NotImplementedError
    def processed(self, st): raise NotImplementedError
    def aligned(self, st): raise NotImplementedError
    def commit_tokens(self, st, n): raise NotImplementedError
    def copy_storage(self, st): raise NotImplementedError
    def leaves(self, st): raise NotImplementedError
    def replace(self, st, caches): raise NotImplementedError
    def copy_cache(self, c): raise NotImplementedError
    def is_trimmable(self, c): raise NotImplementedError
    def mask_array(self, cache, n, window): raise NotImplementedError  # numpy bool array or a mode string


WIDTH = 8  # KVCacheRoundTests.swift:33


def fill(be, cache, lo, hi, one_by_one=True):
    if one_by_one:
        for p in range(lo, hi):
            be.update(cache, *be.kv(p, p + 1))
    else:
        be.update(cache, *be.kv(lo, hi))


def stage(be, rnd, lo, hi):
    k, v = be.kv(lo, hi)
    return [be.update(c, k, v) for c in be.caches_of(rnd)]


def snapshot(be, cache):
    return [a.copy() for a in be.state(cache)], cache.offset, list(be.meta(cache))


def assert_unchanged(be, cache, snap, note):
    arrays, offset, meta = snap
    now = be.state(cache)
    assert len(now) == len(arrays), note
    for a, b in zip(arrays, now):
        assert a.shape == b.shape and np.array_equal(a, b), note
    assert cache.offset == offset, note
    assert be.meta(cache) == meta, note


# ---- invariant 1: the live ring is untouched until commit (KVCacheRoundTests.swift:99-133)
def case_ring_untouched_before_commit(be):
    live = be.rotating(8)
    fill(be, live, 0, 20)
    snap = snapshot(be, live)
    st = be.storage([live])
    rnd = be.begin(st, WIDTH)
    assert rnd is not None
    stage(be, rnd, 20, 24)
    assert_unchanged(be, live, snap, "after staging a full round")
    be.commit(st, rnd, 0)
    assert_unchanged(be, live, snap, "after rolling the round back")


def case_write_through_restored_by_rollback(be):
    live = be.simple()
    fill(be, live, 0, 6)
    st = be.storage([live])
    rnd = be.begin(st, WIDTH)
    stage(be, rnd, 6, 10)
    assert live.offset == 10
    be.commit(st, rnd, 0)
    assert live.offset == 6


# ---- invariant 2: the presentation is the live write path's (KVCacheRoundTests.swift:135-187)
def case_presentation_equals_live_write_path(be):
    window = 8
    staged, written = be.rotating(window), be.rotating(window)
    fill(be, staged, 0, 20)
    fill(be, written, 0, 20)
    st = be.storage([staged])
    rnd = be.begin(st, WIDTH)
    adapter = be.caches_of(rnd)[0]
    assert be.is_staged(adapter)
    m_overlay = be.mask_array(adapter, 4, window)
    m_live = be.mask_array(written, 4, window)
    k, v = be.kv(20, 24)
    pk, pv = be.update(adapter, k, v)
    rk, rv = be.update(written, k, v)
    assert be.positions(pk) == be.positions(rk) == list(range(13, 24))
    assert [-p for p in be.positions(pv)] == be.positions(rk)
    assert isinstance(m_overlay, np.ndarray) and isinstance(m_live, np.ndarray)
    assert m_overlay.shape == m_live.shape and m_overlay.shape[-1] == len(be.positions(pk))
    assert np.array_equal(m_overlay, m_live)
    be.commit(st, rnd, 0)


# ---- invariant 3: commit equivalence (KVCacheRoundTests.swift:228-331)
COMMIT_SCHEDULES = {
    "accepts_nothing": dict(window=8, keep=0, prefill=6, rounds=[(4, 0)] * 3),
    "accepts_everything": dict(window=8, keep=0, prefill=6, rounds=[(4, 4)] * 6),
    "partial_across_wrap": dict(window=8, keep=0, prefill=7,
                                rounds=[(4, 1), (4, 4), (4, 0), (4, 2), (4, 3), (4, 1), (4, 4), (4, 2), (4, 0), (4, 3)]),
    "pinned_prefix": dict(window=8, keep=2, prefill=6, rounds=[(4, 2), (4, 4), (4, 1), (4, 3), (4, 0), (4, 4)]),
    "from_empty": dict(window=8, keep=0, prefill=0, rounds=[(4, 3), (4, 4), (4, 1), (4, 4), (4, 2)]),
    "round_exceeds_window_a": dict(window=4, keep=0, prefill=3, rounds=[(6, 2), (6, 6), (6, 0), (6, 3)]),
    "round_exceeds_window_b": dict(window=4, keep=0, prefill=0, rounds=[(8, 5), (8, 8), (8, 1)]),
}


def case_commit_equivalence(be, window, keep, prefill, rounds):
    live, ref = be.rotating(window, keep), be.rotating(window, keep)
    if prefill:
        fill(be, live, 0, prefill, one_by_one=False)
        fill(be, ref, 0, prefill, one_by_one=False)
    nxt = prefill
    for i, (written, accepted) in enumerate(rounds):
        st = be.storage([live])
        rnd = be.begin(st, WIDTH)
        assert rnd is not None
        stage(be, rnd, nxt, nxt + written)
        be.commit(st, rnd, accepted)
        if accepted:
            be.update(ref, *be.kv(nxt, nxt + accepted))
        nxt += accepted
        assert live.offset == ref.offset, f"round {i}"
        lv, rv = be.view(live, window), be.view(ref, window)
        if lv is None or rv is None:
            assert lv is None and rv is None, f"round {i}"
            continue
        assert be.positions(lv[0]) == be.positions(rv[0]), f"round {i}"
        assert [-p for p in be.positions(lv[1])] == be.positions(rv[0]), f"round {i}"
        assert be.meta(live) == be.meta(ref), f"round {i}"


# ---- mixed topologies (KVCacheRoundTests.swift:333-355)
def case_every_layer_advances_by_accepted(be):
    cache = [be.simple(), be.rotating(8), be.simple(), be.rotating(8)]
    k, v = be.kv(0, 7)
    for c in cache:
        be.update(c, k, v)
    assert {c.offset for c in cache} == {7}
    st = be.storage(cache)
    for accepted in (2, 4, 0, 3):
        before = cache[0].offset
        rnd = be.begin(st, WIDTH)
        stage(be, rnd, 100, 104)
        be.commit(st, rnd, accepted)
        assert {c.offset for c in cache} == {before + accepted}


# ---- adapter surface (KVCacheRoundTests.swift:455-503)
def case_adapter_surface(be):
    live = be.rotating(8)
    st = be.storage([live])
    rnd = be.begin(st, WIDTH)
    adapter = be.caches_of(rnd)[0]
    k, v = be.kv(0, 3)
    pk, pv = be.update(adapter, k, v)
    assert tuple(pk.shape) == tuple(k.shape) and tuple(pv.shape) == tuple(v.shape)
    assert live.offset == 0, "staging the first rows must not initialize the live ring"
    be.commit(st, rnd, 0)

    live = be.rotating(8)
    fill(be, live, 0, 5, one_by_one=False)
    st = be.storage([live])
    rnd = be.begin(st, WIDTH)
    adapter = be.caches_of(rnd)[0]
    assert adapter.offset == 5 and adapter.max_size == 8
    assert adapter.is_trimmable is False and adapter.trim(3) == 0 and live.offset == 5
    stage(be, rnd, 5, 9)
    assert be.staged_count(adapter) == 4 and adapter.offset == 9 and live.offset == 5
    be.commit(st, rnd, 2)
    assert be.staged_count(adapter) == 0 and live.offset == 7


# ---- a staged round vs an accepted-only replay (KVCacheRoundTests.swift:530-668)
def assert_storages_equivalent(be, staged, replayed, note):
    assert be.processed(staged) == be.processed(replayed), note
    assert be.aligned(staged) and be.aligned(replayed), note
    la, lb = be.leaves(staged), be.leaves(replayed)
    assert len(la) == len(lb)
    for i, (a, b) in enumerate(zip(la, lb)):
        assert a.offset == b.offset, f"{note}: leaf {i} offset"
        if a.max_size is not None:
            av, bv = be.view(a, a.max_size), be.view(b, b.max_size)
            if av is None or bv is None:
                assert av is None and bv is None, f"{note}: leaf {i}"
                continue
            assert be.positions(av[0]) == be.positions(bv[0]), f"{note}: leaf {i} window"
            assert be.meta(a) == be.meta(b), f"{note}: leaf {i} ring layout"
        else:
            sa, sb = be.state(a), be.state(b)
            assert len(sa) == len(sb)
            for x, y in zip(sa, sb):
                assert x.shape == y.shape and np.array_equal(x, y), f"{note}: leaf {i} state"


def gemma_storage(be, window, keep):
    return be.storage([be.simple(), be.rotating(window, keep)])


REPLAY_SCHEDULES = {
    "from_empty": dict(window=8, keep=0, prefill=0, rounds=[(4, 3), (4, 4), (4, 1), (4, 4), (4, 2)]),
    "across_wrap": dict(window=8, keep=0, prefill=7,
                        rounds=[(4, 1), (4, 4), (4, 0), (4, 2), (4, 3), (4, 1), (4, 4), (4, 2), (4, 0), (4, 3)]),
    "pinned_prefix": dict(window=8, keep=2, prefill=6, rounds=[(4, 2), (4, 4), (4, 1), (4, 3), (4, 0), (4, 4)]),
    "wider_than_window": dict(window=4, keep=0, prefill=3, rounds=[(6, 2), (6, 6), (6, 0), (6, 3)]),
}


def case_round_matches_accepted_only_replay(be, window, keep, prefill, rounds):
    live = gemma_storage(be, window, keep)
    if prefill:
        k, v = be.kv(0, prefill)
        for leaf in be.leaves(live):
            be.update(leaf, k, v)
        be.commit_tokens(live, prefill)
    nxt = prefill
    for i, (written, retaining) in enumerate(rounds):
        oracle = be.copy_storage(live)
        rnd = be.begin(live, WIDTH)
        assert rnd is not None
        stage(be, rnd, nxt, nxt + written)
        be.commit(live, rnd, retaining)
        if retaining:
            k, v = be.kv(nxt, nxt + retaining)
            for leaf in be.leaves(oracle):
                be.update(leaf, k, v)
            be.commit_tokens(oracle, retaining)
        nxt += retaining
        assert_storages_equivalent(be, live, oracle, f"round {i}")


def case_timeline_aligned(be):
    live = gemma_storage(be, 8, 0)
    k, v = be.kv(0, 5)
    for leaf in be.leaves(live):
        be.update(leaf, k, v)
    be.commit_tokens(live, 5)
    rnd = be.begin(live, WIDTH)
    stage(be, rnd, 5, 9)
    be.commit(live, rnd, 2)
    assert be.processed(live) == 7 and be.aligned(live)


# ---- taking back committed positions (KVCacheRoundTests.swift:670-826)
REWIND_CASES = (
    [dict(window=8, keep=0, prefill=20, written=4, retaining=4, rewinding=r) for r in (1, 2, 3, 4)]
    + [dict(window=32, keep=0, prefill=4, written=4, retaining=4, rewinding=r) for r in (1, 2, 3)]
    + [dict(window=8, keep=2, prefill=20, written=4, retaining=3, rewinding=2),
       dict(window=8, keep=0, prefill=20, written=4, retaining=3, rewinding=3)]
)


def case_rewind_matches_emitted_only_replay(be, window, keep, prefill, written, retaining, rewinding):
    live = gemma_storage(be, window, keep)
    if prefill:
        k, v = be.kv(0, prefill)
        for leaf in be.leaves(live):
            be.update(leaf, k, v)
        be.commit_tokens(live, prefill)
    oracle = be.copy_storage(live)
    rnd = be.begin(live, written)
    stage(be, rnd, prefill, prefill + written)
    be.commit(live, rnd, retaining)
    rewound = be.rewind(live, rewinding)
    assert rewound == min(rewinding, retaining)
    emitted = retaining - rewound
    if emitted:
        k, v = be.kv(prefill, prefill + emitted)
        for leaf in be.leaves(oracle):
            be.update(leaf, k, v)
        be.commit_tokens(oracle, emitted)
    assert_storages_equivalent(be, live, oracle, f"rewind {rewinding} of {retaining}")


def case_rewind_refused_after_another_write(be):
    live = gemma_storage(be, 8, 0)
    k, v = be.kv(0, 20)
    for leaf in be.leaves(live):
        be.update(leaf, k, v)
    be.commit_tokens(live, 20)
    rnd = be.begin(live, 4)
    stage(be, rnd, 20, 24)
    be.commit(live, rnd, 4)
    assert be.processed(live) == 24
    k, v = be.kv(24, 25)
    for leaf in be.leaves(live):
        be.update(leaf, k, v)
    be.commit_tokens(live, 1)
    assert be.rewind(live, 2) == 0
    assert be.processed(live) == 25 and be.aligned(live)


def case_rewind_reaches_live_ring_when_only_some_wrapped(be):
    narrow, wide = be.rotating(4), be.rotating(16)
    live = be.storage([narrow, wide])
    k, v = be.kv(0, 6)
    for leaf in be.leaves(live):
        be.update(leaf, k, v)
    be.commit_tokens(live, 6)
    assert not be.is_trimmable(narrow) and be.is_trimmable(wide)
    oracle = be.copy_storage(live)
    rnd = be.begin(live, 3)
    stage(be, rnd, 6, 9)
    be.commit(live, rnd, 3)
    assert be.rewind(live, 2) == 2
    k, v = be.kv(6, 7)
    for leaf in be.leaves(oracle):
        be.update(leaf, k, v)
    be.commit_tokens(oracle, 1)
    assert_storages_equivalent(be, live, oracle, "mixed-width rewind")


def case_rewind_refused_after_replacement(be):
    original = be.rotating(8)
    live = be.storage([original])
    be.update(original, *be.kv(0, 20))
    be.commit_tokens(live, 20)
    rnd = be.begin(live, 4)
    stage(be, rnd, 20, 24)
    be.commit(live, rnd, 4)
    assert be.processed(live) == 24
    replacement = be.copy_cache(original)
    snap = snapshot(be, replacement)
    be.replace(live, [replacement])
    assert be.rewind(live, 2) == 0
    assert be.processed(live) == 24 and be.aligned(live)
    assert_unchanged(be, replacement, snap, "after a rewind against a replaced entry")


def case_long_random_schedule(be):
    """A long seeded schedule (rounds of random width and acceptance, single-token writes in
    between, a pinned prefix) against an accepted-only replay: exercises slot reuse and, on
    the device, compaction of a fragmented page store."""
    rng = np.random.default_rng(7)
    window, keep = 48, 3
    live, ref = be.rotating(window, keep), be.rotating(window, keep)
    fill(be, live, 0, 11, one_by_one=False)
    fill(be, ref, 0, 11, one_by_one=False)
    nxt = 11
    st = be.storage([live])
    for i in range(160):
        if rng.integers(0, 3) == 0:
            k, v = be.kv(nxt, nxt + 1)
            be.update(live, k, v)
            be.update(ref, k, v)
            be.commit_tokens(st, 1)
            nxt += 1
            continue
        written = int(rng.integers(1, 9))
        accepted = int(rng.integers(0, written + 1))
        rnd = be.begin(st, written)
        pk, pv = stage(be, rnd, nxt, nxt + written)[0]
        got = be.positions(pk)
        assert got[-written:] == list(range(nxt, nxt + written)), f"step {i}"
        assert [-p for p in be.positions(pv)] == got, f"step {i}"
        be.commit(st, rnd, accepted)
        if accepted:
            be.update(ref, *be.kv(nxt, nxt + accepted))
        nxt += accepted
        assert live.offset == ref.offset == nxt, f"step {i}"
        assert be.meta(live) == be.meta(ref), f"step {i}"
        lv, rv = be.view(live, window), be.view(ref, window)
        assert be.positions(lv[0]) == be.positions(rv[0]), f"step {i}"
        assert [-p for p in be.positions(lv[1])] == be.positions(rv[0]), f"step {i}"


SIMPLE_CASES = [
    case_long_random_schedule,
    case_ring_untouched_before_commit,
    case_write_through_restored_by_rollback,
    case_presentation_equals_live_write_path,
    case_every_layer_advances_by_accepted,
    case_adapter_surface,
    case_timeline_aligned,
    case_rewind_refused_after_another_write,
    case_rewind_reaches_live_ring_when_only_some_wrapped,
    case_rewind_refused_after_replacement,
]
