"""The oracle's speculative-round machinery against the known answers of the
reference's KVCacheRoundTests.swift (CPU only)."""
import numpy as np
import pytest

from oracle import kv_oracle as O
from oracle import kv_rounds as R
from tests import rounds_cases as RC


class OracleBackend(RC.Backend):
    def rotating(self, max_size, keep=0):
        return O.RotatingKVCache(max_size, keep=keep)

    def simple(self):
        return O.KVCacheSimple()

    def storage(self, caches):
        return R.Storage(caches)

    def kv(self, lo, hi):
        p = np.arange(lo, hi, dtype=np.float32)
        k = np.broadcast_to(p[None, None, :, None], (1, 1, hi - lo, 2)).copy()
        return k, -k

    def update(self, cache, k, v):
        return cache.update(k, v)

    def positions(self, keys):
        return [int(x) for x in np.asarray(keys)[0, 0, :, 0]]

    def view(self, cache, tail):
        return cache.logical_view(tail)

    def meta(self, cache):
        return cache.get_meta_state()

    def state(self, cache):
        return [np.asarray(a) for a in cache.get_state()]

    def is_staged(self, cache):
        return isinstance(cache, O.RotatingStagedKVCache)

    def staged_count(self, cache):
        return cache.staged_count

    def begin(self, st, width):
        return st.begin_round(width)

    def caches_of(self, rnd):
        return [s.presented for s in rnd]

    def commit(self, st, rnd, n):
        return st.commit(rnd, n)

    def rewind(self, st, n):
        return st.rewind_last_round(n)

    def processed(self, st):
        return st.processed

    def aligned(self, st):
        return st.aligned()

    def commit_tokens(self, st, n):
        st.commit_processed_tokens(n)

    def copy_storage(self, st):
        return st.copy()

    def leaves(self, st):
        return st.cache

    def replace(self, st, caches):
        st.replace(caches)

    def copy_cache(self, c):
        return c.copy()

    def is_trimmable(self, c):
        return c.is_trimmable

    def mask_array(self, cache, n, window):
        m = cache.make_mask(n, window, False)
        return np.asarray(m.array) if m.mode == "array" else m.mode


BE = OracleBackend()


@pytest.mark.parametrize("case", RC.SIMPLE_CASES, ids=lambda f: f.__name__)
def test_round_case(case):
    case(BE)


@pytest.mark.parametrize("name", sorted(RC.COMMIT_SCHEDULES))
def test_commit_equivalence(name):
    RC.case_commit_equivalence(BE, **RC.COMMIT_SCHEDULES[name])


@pytest.mark.parametrize("name", sorted(RC.REPLAY_SCHEDULES))
def test_round_matches_accepted_only_replay(name):
    RC.case_round_matches_accepted_only_replay(BE, **RC.REPLAY_SCHEDULES[name])


@pytest.mark.parametrize("kw", RC.REWIND_CASES, ids=lambda kw: "w{window}k{keep}p{prefill}r{retaining}x{rewinding}".format(**kw))
def test_rewind_matches_emitted_only_replay(kw):
    RC.case_rewind_matches_emitted_only_replay(BE, **kw)


def test_round_refusals():
    # KVCacheRoundTests.swift:357-370, :400-415: a leaf that cannot be rewound refuses the round
    class Probe:
        def __init__(self, trimmable):
            self.offset, self.trimmable = 0, trimmable
        max_size = None

        def is_trimmable_after(self, n):
            return self.trimmable

        @property
        def is_trimmable(self):
            return self.trimmable

        def update(self, k, v):
            self.offset += k.shape[2]
            return k, v

        def trim(self, n):
            t = min(n, self.offset) if self.trimmable else 0
            self.offset -= t
            return t

    good = Probe(True)
    st = R.Storage([good])
    rnd = st.begin_round(8)
    assert rnd is not None and rnd[0].presented is good
    good.update(*BE.kv(0, 4))
    st.commit(rnd, 1)
    assert good.offset == 1
    assert R.Storage([Probe(False)]).begin_round(8) is None
    # quantized layers are written through (KVCacheRoundTests.swift:392-398)
    q = O.QuantizedKVCache(64, 4)
    rnd = R.Storage([q]).begin_round(8)
    assert rnd is not None and rnd[0].presented is q
