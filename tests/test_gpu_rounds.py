"""Speculative rounds on the device (staged rows in spare slots of the ring's page
store, zero-concatenation presentation, commit through the normal write path) against
the known answers of the reference's KVCacheRoundTests.swift -- the same cases the CPU
oracle passes in tests/test_oracle_rounds.py -- plus attention through a staged round
against the oracle."""
import numpy as np
import pytest
import torch

import kvhip
from oracle import kv_oracle as O
from tests import rounds_cases as RC
from tests.util import dev, err_stats, np32, randn

pytestmark = pytest.mark.gpu


class DeviceBackend(RC.Backend):
    dtype = torch.float16

    def rotating(self, max_size, keep=0):
        return kvhip.RotatingKVCache(max_size, keep=keep)

    def simple(self):
        return kvhip.KVCacheSimple()

    def storage(self, caches):
        return kvhip.KVCacheStorage(caches)

    def kv(self, lo, hi):
        p = np.arange(lo, hi, dtype=np.float32)
        k = np.broadcast_to(p[None, None, :, None], (1, 1, hi - lo, 2)).copy()
        return dev(k, self.dtype), dev(-k, self.dtype)

    def update(self, cache, k, v):
        return cache.update(k, v)

    def positions(self, keys):
        return [int(x) for x in np32(keys)[0, 0, :, 0]]

    def view(self, cache, tail):
        return cache.logical_view(tail)

    def meta(self, cache):
        return cache.meta_state

    def state(self, cache):
        return [np32(a) for a in cache.state]

    def is_staged(self, cache):
        return isinstance(cache, kvhip.RotatingStagedKVCache)

    def staged_count(self, cache):
        return cache.staged_count

    def begin(self, st, width):
        return st.begin_round(width)

    def caches_of(self, rnd):
        return rnd.caches

    def commit(self, st, rnd, n):
        return st.commit(rnd, n)

    def rewind(self, st, n):
        return st.rewind_last_round(n)

    def processed(self, st):
        return st.processed_token_count

    def aligned(self, st):
        return st.native_attention_offsets_are_aligned

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
        if m.array is not None:
            return m.array.cpu().numpy()
        return m.mode


BE = DeviceBackend()


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


def test_round_refusals_and_wrapper_errors():
    # a quantized layer is written through (KVCacheRoundTests.swift:392-398)
    q = kvhip.QuantizedKVCache(64, 4)
    rnd = kvhip.KVCacheStorage([q]).begin_round(8)
    assert rnd is not None and rnd.caches[0] is q
    # nested topologies are refused (KVCacheRoundTests.swift:365-370)
    assert kvhip.KVCacheStorage([[kvhip.KVCacheSimple(), kvhip.RotatingKVCache(8)]]).begin_round(8) is None
    # only a ring stages; a second round on the same ring is refused; the wrapper is round-scoped
    L = kvhip.load()
    s = kvhip.KVCacheSimple()
    assert L.kvhip_cache_stage_begin(s._h) < 0
    ring = kvhip.RotatingKVCache(8)
    ring.update(*BE.kv(0, 5))
    st = kvhip.RotatingStagedKVCache(ring)
    assert L.kvhip_cache_stage_begin(ring._h) < 0
    with pytest.raises(RuntimeError):
        st.copy()
    with pytest.raises(RuntimeError):
        st.state = []
    with pytest.raises(kvhip.KVHipError):
        ring.copy()           # the handle refuses too while the round is open
    st.update(*BE.kv(5, 8))
    assert st.offset == 8 and ring.offset == 5 and ring.idx == 5
    k, _ = st.staged_arrays
    assert BE.positions(k) == [5, 6, 7]
    st.commit(1)
    assert ring.offset == 6 and L.kvhip_cache_stage_is_open(ring._h) == 0
    assert L.kvhip_cache_stage_commit(ring._h, 0, None) < 0


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("window,keep,history,queries", [(8, 0, 20, 4), (64, 4, 150, 5), (512, 0, 700, 8), (256, 0, 100, 4)])
def test_staged_attention_matches_logical_order_reference(dtype, window, keep, history, queries):
    """KVCacheRoundTests.swift:189-226: attention through a staged round, past a wrap,
    against a reference that never rotated (the oracle's SDPA over the whole history with
    the causal-and-window mask), max-abs <= 1e-2 and mean-abs <= 1e-3."""
    rng = np.random.default_rng(window + history)
    B, Hq, Hkv, D = 2, 4, 2, 64
    scale = D ** -0.5
    ak, dk = randn(rng, (B, Hkv, history + queries, D), dtype)
    av, dv = randn(rng, (B, Hkv, history + queries, D), dtype)
    aq, dq = randn(rng, (B, Hq, queries, D), dtype)
    live = kvhip.RotatingKVCache(window, keep=keep)
    live.update(dk[:, :, :history - 3].contiguous(), dv[:, :, :history - 3].contiguous(), fetch=False)
    for p in range(history - 3, history):
        live.update(dk[:, :, p:p + 1].contiguous(), dv[:, :, p:p + 1].contiguous(), fetch=False)
    st = kvhip.KVCacheStorage([live])
    rnd = st.begin_round(queries)
    adapter = rnd.caches[0]
    mask = adapter.make_mask(queries, window, False)
    out = adapter.update_attend(dq, dk[:, :, history:].contiguous(), dv[:, :, history:].contiguous(), scale, mask)
    name = {torch.float16: "float16", torch.bfloat16: "bfloat16"}[dtype]
    # the oracle's staged path on the same rows
    olive = O.RotatingKVCache(window, keep=keep, dtype=name)
    olive.update(ak[:, :, :history - 3], av[:, :, :history - 3])
    for p in range(history - 3, history):
        olive.update(ak[:, :, p:p + 1], av[:, :, p:p + 1])
    ost = O.RotatingStagedKVCache(olive)
    omask = ost.make_mask(queries, window, False)
    pk, pv = ost.update(ak[:, :, history:], av[:, :, history:])
    assert adapter.presented_length == pk.shape[2]
    want = O.sdpa(aq, pk, pv, scale, omask, name)
    mx, mean = err_stats(np32(out), want)
    assert mx <= 1e-2 and mean <= 1e-3, (mx, mean)
    if keep == 0:
        qpos = np.arange(history, history + queries)[:, None]
        kpos = np.arange(history + queries)[None, :]
        ref_mask = (qpos >= kpos) & (qpos < kpos + window)
        want = O.sdpa(aq, ak, av, scale, O.Mask("array", ref_mask), name)
        mx, mean = err_stats(np32(out), want)
        assert mx <= 1e-2 and mean <= 1e-3, (mx, mean)
    st.commit(rnd, queries - 1)
    assert live.offset == history + queries - 1
