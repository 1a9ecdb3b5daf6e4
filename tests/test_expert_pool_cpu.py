"""The expert pool's bookkeeping, no GPU (src/zero-tvm/expert-pool.ts:33-148): slot hand-out order, LRU
eviction, pins, the same-request hold, the sizing floor and the hit counters, checked against a small
independent model of an LRU cache."""
import importlib

import numpy as np
import pytest


@pytest.fixture(scope="module")
def ep(pkg):
    return importlib.import_module("zero-tvm_amd.host.expert_pool")


def test_slots_are_handed_out_from_zero_and_pins_come_first(ep):
    p = ep.ExpertPool(4, pin=[99])
    assert p.slot_for(99) == 0 and p.slot_for(5) == -1
    r = p.resolve([5, 7])
    assert list(r.slots) == [1, 2] and r.misses == [(5, 1), (7, 2)] and r.evicted == []
    assert (p.hits, p.requests) == (0, 2)
    r = p.resolve([7, 99, 3])
    assert list(r.slots) == [2, 0, 3] and r.misses == [(3, 3)]
    assert (p.hits, p.requests) == (2, 5) and p.hit_rate == 0.4


def test_lru_eviction_never_takes_a_pin_or_this_requests_own(ep):
    p = ep.ExpertPool(3, pin=[9])
    p.resolve([1])
    p.resolve([2])
    r = p.resolve([3])                     # 1 is the oldest unpinned
    assert r.evicted == [1] and list(r.slots) == [1] and p.slot_for(1) == -1
    r = p.resolve([4, 5])                  # 4 takes 2's slot (oldest), then 5 must not evict 4: takes 3's
    assert r.evicted == [2, 3] and p.slot_for(9) == 0
    assert sorted([p.slot_for(4), p.slot_for(5)]) == [1, 2]
    with pytest.raises(RuntimeError, match="cannot serve this request"):
        p.resolve([6, 7, 8])               # three distinct experts, two unpinned slots


def test_duplicates_share_a_slot_and_load_once(ep):
    p = ep.ExpertPool(2)
    r = p.resolve([4, 4, 4])
    assert list(r.slots) == [0, 0, 0] and r.misses == [(4, 0)] and (p.hits, p.requests) == (2, 3)


def test_floor_and_bad_sizes(ep):
    assert ep.ExpertPool.min_slots(9, 1) == 10 and ep.ExpertPool.min_slots(8) == 8
    with pytest.raises(ValueError, match="at least one slot"):
        ep.ExpertPool(0)
    with pytest.raises(ValueError, match="cannot pin"):
        ep.ExpertPool(1, pin=[1, 2])


def test_against_an_independent_lru_model(ep):
    """Random top-k traffic: residency and hit counts equal those of an ordered-dict LRU with the same
    hold rule; every returned slot really holds the expert asked for."""
    from collections import OrderedDict
    rng = np.random.default_rng(0)
    E, K, SLOTS = 64, 8, 20
    p = ep.ExpertPool(SLOTS, pin=[E])
    lru, hits = OrderedDict(), 0
    held_slots = {E: p.slot_for(E)}
    for _ in range(400):
        req = list(rng.choice(E, K, replace=False)) + [E]
        r = p.resolve(req)
        for e in r.evicted:        # first: an expert can be evicted early in a request and reloaded later in it
            del held_slots[e]
        for e, slot in zip(req, r.slots):
            held_slots[int(e)] = int(slot)
        assert len(set(held_slots.values())) == len(held_slots) <= SLOTS
        now = set()
        for e in req:
            e = int(e)
            if e == E:
                hits += 1
            elif e in lru:
                hits += 1
                lru.move_to_end(e)
            else:
                if len(lru) == SLOTS - 1:
                    victim = next(v for v in lru if v not in now)
                    del lru[victim]
                lru[e] = True
            now.add(e)
        assert set(lru) | {E} == set(held_slots)
    assert p.hits == hits and p.requests == 400 * (K + 1)


def test_slab_strides(ep):
    t = {f: (proj, kind, stride) for f, proj, kind, stride in ep.slab_tensors(2048, 768)}
    assert t["gateWeights"] == ("gate", "w", 768 * 256 * 4) and t["upScales"] == ("up", "s", 768 * 32 * 2)
    assert t["downWeights"] == ("down", "w", 2048 * 96 * 4) and t["downBiases"] == ("down", "b", 2048 * 12 * 2)
    assert len(t) == 9
