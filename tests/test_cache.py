"""The cache's bookkeeping: no slot or block is lost, held twice or freed twice (no GPU)."""
import random

import pytest
import torch

from longbow_quarrel_amd.cache import BLOCK_SIZE, CacheFull, CacheManager, FreeList, blocks_for
from longbow_quarrel_amd.parts.base import KVNeed, StateNeed

CPU = torch.device("cpu")


def test_free_list_gives_each_id_once_and_refuses_double_frees():
    fl = FreeList(4, "slot")
    got = [fl.take() for _ in range(4)]
    assert got == [0, 1, 2, 3] and fl.free_count == 0
    with pytest.raises(CacheFull):
        fl.take()
    fl.give(2)
    with pytest.raises(ValueError):
        fl.give(2)
    with pytest.raises(ValueError):
        fl.give(9)
    assert fl.take() == 2  # given back, used again
    fl.give(3)
    fl.give(0)
    assert fl.take() == 0 and fl.take() == 3


def manager(max_tokens=640, max_slots=4, needs=None):
    needs = needs or {0: KVNeed(2, 16), 1: KVNeed(2, 16)}
    return CacheManager(needs, max_tokens, max_slots, torch.float32, CPU)


def owned_blocks(cm):
    out = []
    for g in cm.kv_groups:
        out.append([b for slot in range(cm.max_slots) for b in g.owned[slot] if b is not None])
    return out


def test_blocks_follow_lengths_and_go_back_on_release():
    cm = manager()
    assert cm.n_blocks == 10 and len(cm.kv_groups) == 1  # layers with the same need share one group
    a, b = cm.acquire(), cm.acquire()
    cm.reserve({a: 65, b: 1})
    cm.advance({a: 65, b: 1})
    g = cm.kv_groups[0]
    assert len(g.owned[a]) == 2 and len(g.owned[b]) == 1 and g.blocks.taken_count == 3
    assert g.table_dev[a, :2].tolist() == g.owned[a] and cm.tokens_held() == 3 * BLOCK_SIZE
    cm.reserve({a: 62})  # up to 127: still two blocks
    cm.advance({a: 62})
    assert g.blocks.taken_count == 3
    cm.reserve({a: 2})
    cm.advance({a: 2})
    assert len(g.owned[a]) == 3 and cm.length(a) == 129
    cm.release(a)
    assert g.blocks.taken_count == 1 and g.owned[a] == []
    with pytest.raises(ValueError):
        cm.release(a)
    with pytest.raises(ValueError):
        cm.length(a)
    c = cm.acquire()
    assert c == a and cm.length(c) == 0  # the slot is used again, empty


def test_a_full_cache_is_an_error_that_changes_nothing():
    cm = manager(max_tokens=256, max_slots=4)
    a, b = cm.acquire(), cm.acquire()
    cm.reserve({a: 128, b: 64})
    cm.advance({a: 128, b: 64})
    before = owned_blocks(cm)
    with pytest.raises(CacheFull):
        cm.reserve({a: 1, b: 65})  # needs 3 more blocks, 1 is free
    assert owned_blocks(cm) == before and cm.kv_groups[0].blocks.free_count == 1
    cm.reserve({a: 1})
    for _ in range(4):
        cm.acquire() if cm.slots.free_count else None
    with pytest.raises(CacheFull):
        cm.acquire()


def test_groups_with_different_needs_have_storage_of_their_own():
    needs = {0: KVNeed(2, 16), 1: KVNeed(2, 16, window=100), 2: KVNeed(1, 32), 3: StateNeed((5,)), 4: KVNeed(2, 16)}
    cm = manager(max_tokens=1280, needs=needs)
    assert len(cm.kv_groups) == 3 and len(cm.state_groups) == 1
    assert sorted(g.layers for g in cm.kv_groups) == [[0, 4], [1], [2]]
    views = cm.layer_views()
    assert views[0].k.shape == (20, 2, BLOCK_SIZE, 16) and views[0].v.shape == (20, 2, 16, BLOCK_SIZE)
    assert views[2].k.shape == (20, 1, BLOCK_SIZE, 32) and views[3].state.shape == (cm.max_slots, 5)
    assert views[0].k.data_ptr() != views[4].k.data_ptr() != views[1].k.data_ptr()
    s = cm.acquire()
    cm.reserve({s: 500})
    cm.advance({s: 500})
    full = next(g for g in cm.kv_groups if g.layers == [0, 4])
    win = next(g for g in cm.kv_groups if g.layers == [1])
    assert full.blocks.taken_count == 8
    # the windowed group keeps the blocks that positions 401.. can still reach, i.e. from block 6 on
    assert [b is not None for b in win.owned[s]] == [False] * 6 + [True, True] and win.blocks.taken_count == 2
    cm.release(s)
    assert full.blocks.taken_count == 0 and win.blocks.taken_count == 0


def test_state_is_cleared_when_a_slot_is_taken():
    cm = manager(needs={0: StateNeed((3,)), 1: KVNeed(1, 16)})
    s = cm.acquire()
    cm.layer_views()[0].state[s] += 7.0
    cm.release(s)
    t = cm.acquire()
    assert t == s and float(cm.layer_views()[0].state[t].abs().sum()) == 0.0


def test_random_traffic_never_loses_or_duplicates_anything():
    rng = random.Random(5)
    cm = manager(max_tokens=64 * 40, max_slots=6, needs={0: KVNeed(1, 16), 1: KVNeed(1, 16, window=70)})
    live = {}
    for step in range(600):
        op = rng.random()
        if op < 0.25 and cm.slots.free_count:
            s = cm.acquire()
            assert s not in live
            live[s] = 0
        elif op < 0.4 and live:
            s = rng.choice(list(live))
            cm.release(s)
            del live[s]
        elif live:
            grow = {s: rng.choice([1, 1, 1, 30, 90]) for s in rng.sample(list(live), rng.randint(1, len(live)))}
            try:
                cm.reserve(grow)
            except CacheFull:
                continue
            cm.advance(grow)
            for s, n in grow.items():
                live[s] += n
        for g in cm.kv_groups:
            held = [b for slot in range(cm.max_slots) for b in g.owned[slot] if b is not None]
            assert len(held) == len(set(held)) == g.blocks.taken_count  # none held twice, none lost
            assert all(g.blocks.is_taken(b) for b in held)
            for s in range(cm.max_slots):
                if s not in live:
                    assert g.owned[s] == []
        for s, n in live.items():
            assert cm.length(s) == n
            assert len(cm.kv_groups[0].owned[s]) == blocks_for(n)
    for s in list(live):
        cm.release(s)
    assert all(g.blocks.taken_count == 0 for g in cm.kv_groups) and cm.slots.taken_count == 0
