"""CPU tests of ExpertCache.load_experts' scheduling (reference src/expert_cache.py:120-201): the device side is
replaced by a stand-in whose copies happen at once, so a copy that is started into a slot before the expert living
there has been handed out shows up as a wrong slab in the caller's hands."""
import itertools

import numpy as np
import pytest
import torch

from mixtral_offloading_amd.expert_cache import ExpertCache
from oracle import hqq_oracle as o

SLAB = 64


class _Module:
    def __init__(self):
        self.storage = torch.UntypedStorage(SLAB)


class _Event:
    busy = False  # what query() reports: the tests of speculative loads set it on the class

    def record(self, stream=None):
        pass

    def query(self):
        return not _Event.busy


class _Stream:
    def wait_event(self, event):
        pass


class HostOnlyCache(ExpertCache):
    """ExpertCache whose streams and events do nothing and whose copies are synchronous host copies."""

    def _init_device_side(self):
        self.copy_stream = _Stream()
        self.ready = [_Event() for _ in self.slots]
        self.released = [_Event() for _ in self.slots]

    def _compute_stream(self):
        return _Stream()

    def _alloc_host(self, nbytes):
        return torch.empty(nbytes, dtype=torch.uint8)

    def _copy_in(self, info, slot):
        torch.as_tensor(self.slots[slot].storage, dtype=torch.uint8).copy_(info.host_slab)
        self._inflight.add(slot)


def _slab_of(e):
    s = torch.UntypedStorage(SLAB)
    torch.as_tensor(s, dtype=torch.uint8).fill_(e + 1)
    return s


def _cache(main, buffers, n=8):
    c = HostOnlyCache(_Module, main_size=main, offload_size=n - main, buffer_size=buffers)
    c._busy_share = 0.0  # (the tests of speculative loads start from a link that has been idle)
    for e in range(n):  # the last `main` experts are resident, as build_model places them
        c.add_expert_storage((0, e), _slab_of(e), eviction_group=0, offload=e < n - main)
    return c


def _content(module):
    return int(torch.as_tensor(module.storage, dtype=torch.uint8)[0]) - 1


@pytest.mark.parametrize("buffers", [1, 2, 4])
@pytest.mark.parametrize("unordered", [True, False])
def test_every_yielded_slot_holds_its_expert_when_a_call_asks_for_all_eight(buffers, unordered):
    """Two resident places and eight requested experts (a prompt that activates every expert of a layer): later
    misses of the call evict its own hits and earlier misses."""
    c = _cache(main=2, buffers=buffers)
    lru = o.LruModel(resident=[6, 7], offloaded=[0, 1, 2, 3, 4, 5])
    rng = np.random.default_rng(buffers)
    for step in range(30):
        req = rng.permutation(8).tolist()
        want_order, _ = lru.load(req)
        got = []
        for (layer, e), module in c.load_experts(*[(0, e) for e in req], unordered=unordered):
            assert _content(module) == e, (step, req, got, e)
            got.append(e)
        assert got == (want_order if unordered else req)
        g = c.group_infos[0]
        assert (g.hits, g.misses) == (lru.hits, lru.misses)
        assert sorted(i.index for i in g.members if not i.offloaded) == sorted(lru.main)
        # what the policy calls resident is what the slots hold, and the spares are the other slots
        for i in g.members:
            if not i.offloaded:
                assert _content(c.slots[g.global_slot[g.slot_of(i.index)]]) == i.index
        resident_slots = {g.global_slot[g.slot_of(i.index)] for i in g.members if not i.offloaded}
        assert sorted(resident_slots | set(c.spare)) == list(range(len(c.slots)))


@pytest.mark.parametrize("main,buffers", [(1, 1), (2, 1), (2, 2), (3, 2), (4, 4)])
def test_random_requests_in_both_iteration_orders(main, buffers):
    for unordered in (True, False):
        c = _cache(main=main, buffers=buffers)
        lru = o.LruModel(resident=list(range(8 - main, 8)), offloaded=list(range(8 - main)))
        rng = np.random.default_rng(main * 10 + buffers)
        for step in range(200):
            req = rng.choice(8, size=int(rng.integers(1, 9)), replace=False).tolist()
            lru.load(req)
            for (layer, e), module in c.load_experts(*[(0, e) for e in req], unordered=unordered):
                assert _content(module) == e, (unordered, step, req, e)
            g = c.group_infos[0]
            assert (g.hits, g.misses) == (lru.hits, lru.misses)
            assert sorted(i.index for i in g.members if not i.offloaded) == sorted(lru.main)


def test_all_orders_of_a_small_group():
    """Exhaustive: every ordered request of 1..4 experts out of 4, one resident place, one buffer."""
    for unordered in (True, False):
        for n in range(1, 5):
            for req in itertools.permutations(range(4), n):
                c = _cache(main=1, buffers=1, n=4)
                for _ in range(2):  # the second round starts from what the first one left
                    for (layer, e), module in c.load_experts(*[(0, e) for e in req], unordered=unordered):
                        assert _content(module) == e, (unordered, req, e)


def test_leaving_the_loop_early_still_loads_what_the_policy_counts_as_resident():
    c = _cache(main=2, buffers=2)
    for (layer, e), module in c.load_experts(*[(0, e) for e in (0, 1, 2, 6)], unordered=True):
        break
    assert not c.active
    g = c.group_infos[0]
    for i in g.members:
        if not i.offloaded:
            assert _content(c.slots[g.global_slot[g.slot_of(i.index)]]) == i.index


def test_host_copies_are_pinned_only_for_experts_that_can_be_evicted():
    c = HostOnlyCache(_Module, main_size=4, offload_size=2, buffer_size=1)
    for e in range(2):  # group 0: everything resident, nothing to evict
        c.add_expert_storage((0, e), _slab_of(e), eviction_group=0, offload=False)
    assert all(c.registered_experts[(0, e)].host_slab is None for e in range(2))
    assert int(c.expert_bytes((0, 1))[0]) == 2
    c.add_expert_storage((1, 0), _slab_of(10), eviction_group=1, offload=False)
    assert c.registered_experts[(1, 0)].host_slab is None
    c.add_expert_storage((1, 1), _slab_of(11), eviction_group=1, offload=True)  # group 1 becomes evictable
    assert int(c.registered_experts[(1, 0)].host_slab[0]) == 11
    c.add_expert_storage((1, 2), _slab_of(12), eviction_group=1, offload=False)
    assert c.registered_experts[(1, 2)].host_slab is not None
    assert all(c.registered_experts[(0, e)].host_slab is None for e in range(2))
    for (g, e), module in c.load_experts((1, 1), (1, 0), unordered=True):
        assert _content(module) == 10 + e


def _resident(c):
    g = c.group_infos[0]
    return sorted(m.index for m in g.members if g.slot_of(m.index) >= 0)


def test_a_guess_is_dropped_while_the_host_link_is_busy():
    c = _cache(main=4, buffers=2)  # resident: 4 5 6 7
    for _ in c.load_experts((0, 6), (0, 7), (0, 3)):  # 3 evicts 4; its copy stays "unfinished" below
        pass
    assert _resident(c) == [3, 5, 6, 7]
    _Event.busy = True
    try:
        assert c.prefetch((0, 0), (0, 1)) == 0
        assert _resident(c) == [3, 5, 6, 7] and c.stats()["prefetch_skipped_busy"] == 2 and c.stats()["prefetch_loads"] == 0
        c.prefetch_backlog = 1  # a caller may let guesses queue behind that many unfinished copies
        assert c.prefetch((0, 0)) == 1 and _resident(c) == [0, 3, 6, 7]  # 5 went: 3, 6 and 7 are the latest request's
        c.prefetch_backlog = 0
    finally:
        _Event.busy = False
    # 0 is resident; 1 finds nobody it may evict (3, 6, 7 are protected, 0 belongs to the same guess)
    assert c.prefetch((0, 0), (0, 1)) == 0 and _resident(c) == [0, 3, 6, 7]
    st = c.stats()
    assert st["prefetch_loads"] == 1 and st["prefetch_skipped_protected"] == 1
    assert st["hits"] == 2 and st["misses"] == 1  # guesses are not counted as requests


def test_a_guess_does_not_evict_the_latest_requests_experts_until_guesses_have_proved_better():
    """Two places, top-2 requests: every resident expert belongs to the latest request, so guesses are dropped; once
    enough guesses have been scored and they are right more often than experts repeat, they may evict."""
    c = _cache(main=2, buffers=2)
    for _ in c.load_experts((0, 6), (0, 7)):
        pass
    assert c.prefetch((0, 0), (0, 1)) == 0 and _resident(c) == [6, 7]
    assert c.stats()["prefetch_skipped_protected"] == 2
    # guesses that are always right, requests that never repeat an expert
    seq = [(0, 1), (2, 3), (4, 5), (6, 7), (0, 1), (2, 3)]
    for a, b in seq:
        for (_, e), module in c.load_experts((0, a), (0, b)):
            assert _content(module) == e
        nxt = seq[(seq.index((a, b)) + 1) % len(seq)]
        c.prefetch((0, nxt[0]), (0, nxt[1]))
    st = c.stats()
    assert st["guess_right"] == st["guess_scored"] >= 8 and st["reuse_right"] == 0
    assert st["prefetch_loads"] > 0  # by now guesses evict
    loads = st["prefetch_loads"]
    for (_, e), module in c.load_experts((0, 4), (0, 5)):
        assert _content(module) == e
    assert c.stats()["prefetch_useful"] >= 2 and c.stats()["prefetch_loads"] == loads


def test_a_guess_of_resident_experts_changes_nothing():
    c = _cache(main=4, buffers=2)
    for _ in c.load_experts((0, 4), (0, 5)):
        pass
    assert c.prefetch((0, 6), (0, 7)) == 0  # resident already
    # 6 and 7 are still the least recently used: two misses evict exactly them
    for _ in c.load_experts((0, 0), (0, 1)):
        pass
    assert _resident(c) == [0, 1, 4, 5]


def test_guesses_stop_when_the_link_has_mostly_been_busy():
    """The share of prefetch calls that found unfinished copies is tracked; above the limit no guess is acted on, even
    at a call that finds the link idle, and guesses resume once the link has been idle for a while."""
    c = _cache(main=4, buffers=2)
    for _ in c.load_experts((0, 6), (0, 7), (0, 3)):
        pass
    _Event.busy = True
    try:
        for _ in range(6):
            assert c.prefetch((0, 0)) == 0
    finally:
        _Event.busy = False
    assert c._busy_share > c.prefetch_busy_limit
    assert c.prefetch((0, 0)) == 0  # idle now, but busy at most of the recent calls
    calls = 1
    while c.prefetch((0, 0)) == 0:
        calls += 1
        assert calls < 40
    assert calls > 3 and 0 in _resident(c)
