"""The cache's bookkeeping on the host: no slot or page lost, held twice or freed twice;
reuse; groups with storage of their own; the window's pages; the fixed-size state."""
import random

import pytest
import torch

from minfer_amd.cache import PAGE, Cache, CacheError, CacheFull, KVRequest, PagePool, StateRequest


def make(max_tokens=64 * 8, max_seqs=4, window=None, with_state=False):
    reqs = {0: KVRequest(2, 16), 1: KVRequest(2, 16), 2: KVRequest(1, 32, window=window) if window else KVRequest(2, 16)}
    if with_state:
        reqs[3] = StateRequest((3, 5))
    return Cache(reqs, max_tokens, max_seqs, torch.float32, "cpu")


def test_page_pool_refuses_double_free_and_overdraw():
    pool = PagePool(4)
    a = pool.take(3)
    assert len(set(a)) == 3 and pool.free_pages == 1
    with pytest.raises(CacheFull):
        pool.take(2)
    pool.give(a[:1])
    with pytest.raises(CacheError):
        pool.give(a[:1])
    with pytest.raises(CacheError):
        pool.give([99])
    pool.give(a[1:])
    assert pool.free_pages == 4


def test_groups_have_storage_of_their_own():
    c = make(window=100)
    assert len(c.groups) == 2
    full = c.group_of[0]
    assert c.group_of[1] is full and c.group_of[2] is not full
    assert full.k.shape == (2, 8, 2, PAGE, 16) and c.group_of[2].k.shape == (1, 8, 1, PAGE, 32)
    k0, v0, g = c.kv(0)
    k1, _, _ = c.kv(1)
    assert k0.shape == (8, 2, PAGE, 16) and k0.data_ptr() != k1.data_ptr() and g is full


def test_values_may_have_a_width_of_their_own():
    """An entry may ask for value rows of another width than its key rows: its group's V pages have
    that width (in both layouts), sizing counts it, and the built-in write, which takes one width,
    refuses the entry instead of writing rows of the wrong size."""
    from minfer_amd.engine.engine import cache_bytes_per_token
    reqs = {0: KVRequest(2, 16), 1: KVRequest(2, 16, v_head_dim=24), 2: KVRequest(2, 16, v_head_dim=16)}
    assert reqs[0] != reqs[1] and reqs[1].value_dim == 24 and reqs[0].value_dim == 16
    c = Cache(reqs, 64 * 4, 2, torch.float32, "cpu")
    assert len(c.groups) == 3 or c.group_of[0] is not c.group_of[1]
    k, v, g = c.kv(1)
    assert k.shape == (4, 2, PAGE, 16) and v.shape == (4, 2, PAGE, 24)
    b = Cache(reqs, 64 * 4, 2, torch.bfloat16, "cpu")
    assert b.kv(1)[1].shape == (4, 2, 2, 24, PAGE // 2) and b.kv(0)[1].shape == (4, 2, 2, 16, PAGE // 2)
    assert cache_bytes_per_token(reqs, torch.float32) == (2 * 32 + 2 * 40 + 2 * 32) * 4
    with pytest.raises(CacheError, match="value width of its own"):
        c.store_kv(1, torch.zeros(1, 4 * 16), None, 2, torch.zeros(1, 2 * 16))


def test_slots_are_given_back_and_used_again():
    c = make(max_seqs=2)
    a, b = c.alloc_slot(), c.alloc_slot()
    assert a != b
    with pytest.raises(CacheFull):
        c.alloc_slot()
    c.reserve({a: 70, b: 5})
    c.commit({a: 70, b: 5})
    assert c.length(a) == 70 and c.free_tokens() == (8 - 3) * PAGE
    c.free_slot(a)
    with pytest.raises(CacheError):
        c.free_slot(a)
    with pytest.raises(CacheError):
        c.length(a)
    a2 = c.alloc_slot()
    assert a2 == a and c.length(a2) == 0 and c.free_tokens() == (8 - 1) * PAGE
    c.check_invariants()


def test_reserve_is_all_or_nothing():
    c = make(max_tokens=64 * 4)
    a, b = c.alloc_slot(), c.alloc_slot()
    c.reserve({a: 100})
    with pytest.raises(CacheFull):
        c.reserve({a: 120, b: 200})            # needs 0 + 4 pages, 2 are free
    assert c.free_tokens() == 2 * PAGE and c.group_of[0].pages[b] == []
    c.reserve({b: 128})
    assert c.free_tokens() == 0
    c.check_invariants()


def test_reserve_below_length_is_an_error():
    c = make()
    a = c.alloc_slot()
    c.reserve({a: 10})
    c.commit({a: 10})
    with pytest.raises(CacheError):
        c.reserve({a: 5})


def test_window_group_gives_pages_back():
    c = make(max_tokens=64 * 8, window=70)
    a = c.alloc_slot()
    win = c.group_of[2]
    c.reserve({a: 300})
    c.commit({a: 300})
    # a query at position >= 300 reads keys > 300 - 70 = 230, i.e. from page 231 // 64 = 3
    assert win.pages[a][:3] == [-1, -1, -1] and all(p >= 0 for p in win.pages[a][3:])
    assert win.pool.free_pages == 8 - 2 and c.group_of[0].pool.free_pages == 8 - 5
    with pytest.raises(CacheError):
        c.truncate(a, 100)                     # the window already dropped what 100 needs
    c.check_invariants()
    c.free_slot(a)
    assert win.pool.free_pages == 8
    c.check_invariants()


def test_truncate_and_state():
    c = make(with_state=True)
    a = c.alloc_slot()
    c.state(3)[a] += 7.0
    c.reserve({a: 130})
    c.commit({a: 130})
    with pytest.raises(CacheError):
        c.truncate(a, 64)                      # fixed-size state cannot be rolled back
    c.free_slot(a)
    b = c.alloc_slot()
    assert b == a and float(c.state(3)[b].abs().sum()) == 0.0      # zeroed when the slot is taken
    c2 = make()
    s = c2.alloc_slot()
    c2.reserve({s: 130})
    c2.commit({s: 130})
    c2.truncate(s, 64)
    assert c2.length(s) == 64 and c2.free_tokens() == 7 * PAGE
    c2.check_invariants()


def test_random_walk_keeps_every_page_accounted_for():
    rng = random.Random(0)
    c = make(max_tokens=64 * 16, max_seqs=5, window=90, with_state=True)
    live = {}
    for _ in range(600):
        op = rng.random()
        if op < 0.25 and len(live) < 5:
            live[c.alloc_slot()] = 0
        elif op < 0.4 and live:
            s = rng.choice(list(live))
            c.free_slot(s)
            del live[s]
        elif live:
            s = rng.choice(list(live))
            n = live[s] + rng.choice([1, 1, 1, 17, 64, 130])
            try:
                c.reserve({s: n})
                c.commit({s: n})
                live[s] = n
            except CacheFull:
                pass
        c.check_invariants()
        assert {s: c.length(s) for s in c.live_slots()} == live
    for s in list(live):
        c.free_slot(s)
    c.check_invariants()
    assert all(g.pool.free_pages == g.pool.n_pages for g in c.groups)
