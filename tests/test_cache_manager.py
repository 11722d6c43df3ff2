"""The cache manager on the host: no page lost, held twice or freed twice, under random
orders of requests; groups with pages of their own; windows give pages back; state slots."""
import random

import pytest
import torch

from swifttransformer_amd.cache import CacheManager, OutOfPages, OutOfSlots, PagePool
from swifttransformer_amd.parts import CacheNeed

FULL = CacheNeed("paged_kv", num_kv_heads=2, head_dim=16)
WIN = CacheNeed("paged_kv", num_kv_heads=2, head_dim=16, window=10)
STATE = CacheNeed("state", state_shape=(4,), state_dtype=torch.float32)


def test_pool_basics():
    pool = PagePool(4)
    a = pool.alloc(3)
    assert a == [0, 1, 2] and pool.num_free == 1
    with pytest.raises(OutOfPages):
        pool.alloc(2)
    assert pool.num_free == 1                    # a failed request takes nothing
    pool.free([1])
    assert pool.alloc(1) == [1]                  # a page given back is the next one handed out
    with pytest.raises(ValueError, match="freed twice"):
        pool.free([3])
    pool.free([0])
    with pytest.raises(ValueError, match="freed twice"):
        pool.free([0])
    with pytest.raises(ValueError, match="not of this pool"):
        pool.free([9])


def test_groups_have_pages_of_their_own():
    m = CacheManager({0: FULL, 1: WIN, 2: FULL, 3: STATE, 4: WIN}, page_size=4,
                     num_pages={0: 8, 1: 5}, max_seqs=3, max_pages_per_seq=16)
    assert [g.cache_ids for g in m.groups] == [[0, 2], [1, 4], [3]]
    assert m.group_of_cache == {0: 0, 2: 0, 1: 1, 4: 1, 3: 2}
    assert [g.index for g in m.paged_groups] == [0, 1]
    m.admit("a")
    m.extend("a", 9)
    assert len(m.requests["a"].tables[0]) == 3 and len(m.requests["a"].tables[1]) == 3
    assert m.num_free_pages(0) == 5 and m.num_free_pages(1) == 2
    m.check_invariants()


def test_window_gives_pages_back_as_it_passes():
    m = CacheManager({0: FULL, 1: WIN}, page_size=4, num_pages=16, max_seqs=2, max_pages_per_seq=32)
    m.admit("a")
    length = 0
    for step in range(40):
        m.release_behind_window("a", length)
        m.extend("a", length + 1)
        length += 1
        m.check_invariants()
        t_full, t_win = m.requests["a"].tables[0], m.requests["a"].tables[1]
        assert all(p >= 0 for p in t_full)
        # the token at position length-1 reads positions >= length-1-9: their pages must be held
        first_read = max(0, (length - 1) - 10 + 1)
        for pi, p in enumerate(t_win):
            if pi >= first_read // 4:
                assert p >= 0, (length, pi)
        assert sum(p >= 0 for p in t_win) <= 4          # ceil((10 + 3) / 4) + 1 pages at most
    assert m.num_free_pages(1) >= 12
    m.finish("a")
    assert m.num_free_pages(0) == 16 and m.num_free_pages(1) == 16


def test_extend_is_all_or_nothing_over_groups():
    m = CacheManager({0: FULL, 1: WIN}, page_size=4, num_pages={0: 8, 1: 2}, max_seqs=2, max_pages_per_seq=16)
    m.admit("a")
    with pytest.raises(OutOfPages):
        m.extend("a", 12)           # group 1 has only 2 pages
    assert m.num_free_pages(0) == 8 and m.num_free_pages(1) == 2
    assert m.requests["a"].length == 0
    m.check_invariants()


def test_slots():
    m = CacheManager({0: FULL}, page_size=4, num_pages=8, max_seqs=2, max_pages_per_seq=8)
    a, b = m.admit("a"), m.admit("b")
    assert {a.slot, b.slot} == {0, 1}
    with pytest.raises(OutOfSlots):
        m.admit("c")
    with pytest.raises(KeyError):
        m.admit("a")
    m.finish("a")
    assert m.admit("c").slot == a.slot
    m.check_invariants()


@pytest.mark.parametrize("seed", range(6))
def test_random_lifecycles_conserve_pages(seed):
    rng = random.Random(seed)
    m = CacheManager({0: FULL, 1: WIN, 2: FULL}, page_size=rng.choice([1, 3, 4, 8]),
                     num_pages={0: 40, 1: 12}, max_seqs=5, max_pages_per_seq=64)
    live = {}
    next_id = 0
    for _ in range(600):
        op = rng.random()
        if op < 0.25 and m.num_free_slots > 0:
            m.admit(next_id)
            live[next_id] = 0
            next_id += 1
        elif op < 0.8 and live:
            rid = rng.choice(list(live))
            n = rng.choice([1, 1, 1, 2, 5, 17])
            m.release_behind_window(rid, live[rid])
            try:
                m.extend(rid, live[rid] + n)
                live[rid] += n
            except OutOfPages:
                victim = rng.choice(list(live))
                if rng.random() < 0.5:
                    m.finish(victim)
                    del live[victim]
                else:
                    m.reset_request(victim)
                    live[victim] = 0
            except ValueError:
                m.finish(rid)           # reached the per-request page limit
                del live[rid]
        elif live:
            rid = rng.choice(list(live))
            m.finish(rid)
            del live[rid]
        m.check_invariants()
        for rid, n in live.items():
            assert m.requests[rid].length == n
    for rid in list(live):
        m.finish(rid)
    m.check_invariants()
    assert m.num_free_pages(0) == 40 and m.num_free_pages(1) == 12 and m.num_free_slots == 5


def test_every_admission_fires_the_hooks_with_the_slot():
    """Whoever admits a request (a scheduler, a replay, a re-admission after pre-emption), the
    owner of per-slot device state hears of it and can clear the slot."""
    from swifttransformer_amd.cache.manager import CacheManager
    from swifttransformer_amd.parts import CacheNeed
    m = CacheManager({0: CacheNeed("paged_kv", num_kv_heads=2, head_dim=16),
                      1: CacheNeed("state", state_shape=(4,))}, page_size=4, num_pages=8, max_seqs=2,
                     max_pages_per_seq=4)
    cleared = []
    m.on_admit.append(cleared.append)
    a = m.admit("a").slot
    b = m.admit("b").slot
    m.finish("a")
    c = m.admit("c").slot
    assert cleared == [a, b, c] and c == a          # the slot of a finished request is taken over, and cleared again
    m.check_invariants()
