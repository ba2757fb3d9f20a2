"""The cache manager: no page lost, held twice or freed twice, under random
orders of requests; windows give pages back; state slots."""

import random

import pytest
import torch

from qwen3_from_scratch_amd.cache import CacheManager, OutOfPages, PagePool
from qwen3_from_scratch_amd.parts import CacheNeed
from qwen3_from_scratch_amd.parts.attention import keys_and_values


def test_pool_refuses_double_free_and_overdraw():
    pool = PagePool(3)
    a, b, c = pool.take(), pool.take(), pool.take()
    assert sorted([a, b, c]) == [0, 1, 2]
    with pytest.raises(OutOfPages):
        pool.take()
    pool.give(b)
    with pytest.raises(RuntimeError):
        pool.give(b)
    with pytest.raises(RuntimeError):
        pool.give(7)
    assert pool.take() == b                      # the page freed last is used again first


def test_pages_follow_the_references_arithmetic():
    # test/inference/test_block_manager.py:9-97, block size 16
    m = CacheManager([keys_and_values(2, 8)], page_size=16, num_pages=2, max_requests=4)
    assert not m.can_grow("a", 33)               # 33 tokens need 3 pages, 2 exist
    assert m.can_grow("a", 32)
    m.admit("a")
    m.reserve("a", 16)
    m.commit("a", 16)
    assert len(m.block_table("a", 0)) == 1
    assert m.pages_missing("a", 1) == [1]        # 16 cached + 1 -> a second page
    m.release("a")
    m.admit("b")
    m.reserve("b", 15)
    m.commit("b", 15)
    assert m.pages_missing("b", 1) == [0]        # 15 cached + 1 -> none
    m.release("b")
    assert m.num_free() == 2
    m.audit()


def test_reserve_is_all_or_nothing_across_groups():
    needs = [keys_and_values(2, 8), keys_and_values(2, 8, window=16), keys_and_values(2, 8)]
    m = CacheManager(needs, page_size=8, num_pages=4, max_requests=2)
    assert len(m.groups) == 2 and m.groups[0].planes == [0, 2] and m.groups[1].planes == [1]
    m.admit("a")
    m.reserve("a", 24)
    m.commit("a", 24)
    m.admit("b")
    with pytest.raises(OutOfPages):
        m.reserve("b", 16)                       # group 0 has one page left
    assert m.block_table("b", 0) == [] and m.block_table("b", 1) == []
    m.audit()


def test_window_gives_pages_back_as_it_passes_them():
    m = CacheManager([keys_and_values(1, 8, window=20)], page_size=8, num_pages=6, max_requests=1)
    m.admit("w")
    length = 0
    for n in [5, 9, 1, 1, 30, 2]:
        m.reserve("w", n)
        m.commit("w", n)
        length += n
        table = m.block_table("w", 0)
        first_needed = max(0, length - 20 + 1)   # the next query at `length` sees keys from here
        for blk, page in enumerate(table):
            covered_end = (blk + 1) * 8
            assert (page == -1) == (covered_end <= first_needed), (length, blk, table)
        m.audit()
    assert m.num_free() == 6 - sum(p >= 0 for p in m.block_table("w", 0))
    m.release("w")
    assert m.num_free() == 6


def test_state_slots_are_unique_and_come_back():
    need = CacheNeed(state_shape=(3, 5), state_dtype=torch.float32)
    m = CacheManager([need, need, None], page_size=16, num_pages=0, max_requests=3)
    assert len(m.groups) == 0 and len(m.state_groups) == 1 and m.state_groups[0].planes == [0, 1]
    slots = [m.admit(r) for r in "abc"]
    assert sorted(slots) == [0, 1, 2] and m.fresh_slots == slots
    with pytest.raises(OutOfPages):
        m.admit("d")
    with pytest.raises(KeyError):
        m.admit("a")
    m.release("b")
    assert m.admit("d") == slots[1]
    m.audit()


@pytest.mark.parametrize("seed", range(6))
def test_random_orders_lose_nothing(seed):
    rng = random.Random(seed)
    needs = [keys_and_values(2, 16), keys_and_values(2, 16, window=rng.choice([9, 24, 40])), keys_and_values(2, 16)]
    page = rng.choice([4, 8, 16])
    m = CacheManager(needs, page_size=page, num_pages=rng.randint(6, 20), max_requests=4)
    live, counter = {}, 0
    for _ in range(600):
        roll = rng.random()
        if roll < 0.25 and len(live) < 4:
            rid = "r%d" % counter
            counter += 1
            m.admit(rid)
            live[rid] = 0
        elif roll < 0.85 and live:
            rid = rng.choice(list(live))
            n = rng.choice([1, 1, 1, 2, 3, 7, 16, 33])
            if m.can_grow(rid, n):
                m.reserve(rid, n)
                m.commit(rid, n)
                live[rid] += n
                assert m.length(rid) == live[rid]
                # every position a later query can see has a page
                for g, grp in enumerate(m.groups):
                    table = m.block_table(rid, g)
                    lo = 0 if grp.window == 0 else max(0, live[rid] - grp.window + 1)
                    for pos in range(lo, live[rid]):
                        assert table[pos // page] >= 0
            else:
                with pytest.raises(OutOfPages):
                    m.reserve(rid, n)
        elif live:
            rid = rng.choice(list(live))
            m.release(rid)
            del live[rid]
        m.audit()
    for rid in list(live):
        m.release(rid)
    m.audit()
    assert all(g.pool.num_free == g.pool.num_pages for g in m.groups)


# ---- the prefix index ----

def _run(m, rid, tokens, register=True):
    """Admit, take over what the index has, compute the rest, register; returns tokens taken over."""
    m.admit(rid)
    got = m.share_prefix(rid, tokens)
    m.reserve(rid, len(tokens) - got)
    m.commit(rid, len(tokens) - got)
    if register:
        m.register_prefix(rid, tokens)
    return got


def test_prefix_blocks_are_shared_counted_and_kept_after_their_holders():
    m = CacheManager([keys_and_values(2, 8), keys_and_values(4, 16)], page_size=4, num_pages=10, max_requests=4, prefix_cache=True)
    assert m.prefix_cache and len(m.groups) == 2
    a = list(range(100, 111))                     # 11 tokens: two full blocks and three tokens
    assert _run(m, "a", a) == 0
    assert _run(m, "b", a[:8] + [7, 7, 7]) == 8   # the same two blocks, then its own
    assert m.block_table("b", 0)[:2] == m.block_table("a", 0)[:2] and m.block_table("b", 0)[2] != m.block_table("a", 0)[2]
    assert m.block_table("b", 1)[:2] == m.block_table("a", 1)[:2]
    assert _run(m, "c", a[:8]) == 4               # a whole hit keeps a token to compute: one block only
    assert _run(m, "d", a[:4] + [1] + a[5:]) == 4 # a change in the second block: the first alone is shared
    m.audit()
    assert m.num_free() == 10 - 3 - 1 - 1 - 2     # a: 3 pages, b: 1 more, c: 1 more, d: 2 more
    for rid in "abcd":
        m.release(rid)
        m.audit()
    assert m.num_free() == 10 and m.groups[0].pool.num_free < 10      # the nodes keep their pages, which count as free
    assert _run(m, "e", a) == 8                   # and a later request still finds them
    m.release("e")
    m.forget_prefixes()
    m.audit()
    assert m.groups[0].pool.num_free == 10 and m.groups[1].pool.num_free == 10
    m.admit("f")
    assert m.share_prefix("f", a) == 0


def test_prefix_nodes_are_forgotten_oldest_first_when_pages_run_out():
    m = CacheManager([keys_and_values(2, 8)], page_size=4, num_pages=6, max_requests=3, prefix_cache=True)
    first, second = list(range(10, 18)), list(range(50, 58))
    _run(m, "a", first + [1])
    m.release("a")                                # two idle nodes (and a private page that went back)
    _run(m, "b", second + [1])
    m.release("b")                                # four idle nodes
    assert m.num_free() == 6 and m.groups[0].pool.num_free == 2
    m.admit("c")
    m.reserve("c", 16)                            # four pages: the pool's two, and `first`'s two nodes go
    m.commit("c", 16)
    m.audit()
    m.admit("d")
    assert m.share_prefix("d", first + [1]) == 0 and m.can_grow("d", 8)
    m.release("d")
    m.admit("e")
    assert m.share_prefix("e", second + [1]) == 8   # the younger ones are still there
    assert not m.can_grow("e", 1)                 # c holds four pages, e's nodes two: nothing is idle any more
    with pytest.raises(OutOfPages):
        m.reserve("e", 1)
    m.release("c")
    assert m.can_grow("e", 16)
    m.audit()


def test_prefix_index_stays_off_for_windows_and_state():
    assert not CacheManager([keys_and_values(2, 8, window=16)], 4, 8, 2, prefix_cache=True).prefix_cache
    assert not CacheManager([keys_and_values(2, 8), CacheNeed(state_shape=(3,), state_dtype=torch.float32)], 4, 8, 2,
                            prefix_cache=True).prefix_cache
    m = CacheManager([keys_and_values(2, 8)], 4, 8, 2)
    assert not m.prefix_cache
    m.admit("a")
    assert m.share_prefix("a", list(range(9))) == 0
    m.register_prefix("a", list(range(9)))
    m.audit()


@pytest.mark.parametrize("seed", range(6))
def test_random_orders_with_shared_prefixes_lose_nothing(seed):
    rng = random.Random(seed)
    m = CacheManager([keys_and_values(2, 8), keys_and_values(1, 16)], page_size=4, num_pages=24, max_requests=5, prefix_cache=True)
    stems = [[rng.randrange(5) for _ in range(rng.randrange(4, 20))] for _ in range(3)]
    live = {}                                     # rid -> (tokens, computed)
    count = 0
    for _ in range(600):
        roll = rng.random()
        if roll < 0.3 and len(live) < 5:
            tokens = list(rng.choice(stems))[:rng.randrange(1, 20)] + [rng.randrange(5) for _ in range(rng.randrange(1, 9))]
            rid = "r%d" % count
            count += 1
            m.admit(rid)
            live[rid] = (tokens, m.share_prefix(rid, tokens))
            assert live[rid][1] % 4 == 0 and live[rid][1] < len(tokens)
        elif roll < 0.8 and live:
            rid = rng.choice(sorted(live))
            tokens, computed = live[rid]
            n = rng.randrange(1, 7)
            if computed + n > len(tokens):
                tokens = tokens + [rng.randrange(5) for _ in range(computed + n - len(tokens))]
            if m.can_grow(rid, n):
                m.reserve(rid, n)
                m.commit(rid, n)
                live[rid] = (tokens, computed + n)
                m.register_prefix(rid, tokens)
            else:
                with pytest.raises(OutOfPages):
                    m.reserve(rid, n)
        elif live:
            rid = rng.choice(sorted(live))
            m.release(rid)
            del live[rid]
        m.audit()
        for rid, (tokens, computed) in live.items():
            assert m.length(rid) == computed
    for rid in list(live):
        m.release(rid)
    m.audit()
    assert m.num_free(0) == 24 and m.num_free(1) == 24
    m.forget_prefixes()
    assert all(g.pool.num_free == 24 for g in m.groups)
