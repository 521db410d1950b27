"""The cache manager's bookkeeping, without a GPU: no page lost, held twice or freed twice,
under random orders of requests; windows give pages back; failures change nothing."""

import random

import pytest

from mini_llm_amd.cache import NO_PAGE, CacheError, CacheManager, OutOfPages, PagePool
from mini_llm_amd.models.base import CacheGroupSpec
from mini_llm_amd.parts.base import StateNeed

FULL = CacheGroupSpec("full", (0, 1), 2, 16, None)
WINDOW = CacheGroupSpec("win", (2,), 1, 32, 40)


def manager(groups=(FULL,), num_pages=8, page_size=16, max_requests=4, max_length=None):
    return CacheManager(list(groups), {}, num_pages=num_pages, page_size=page_size, max_requests=max_requests, max_length=max_length)


def test_pool_refuses_double_free_and_overdraw():
    pool = PagePool(3)
    pages = pool.take(2)
    with pytest.raises(OutOfPages):
        pool.take(2)
    assert pool.num_free == 1  # a refused take takes nothing
    pool.give(pages)
    with pytest.raises(RuntimeError, match="not held"):
        pool.give([pages[0]])
    with pytest.raises(RuntimeError, match="not held"):
        pool.give([17])


def test_block_table_grows_with_the_request():
    m = manager()
    m.open("a")
    assert m.pages_needed("a", 1) == [1] and m.pages_needed("a", 16) == [1] and m.pages_needed("a", 17) == [2]
    m.reserve("a", 17); m.commit("a", 17)
    assert m.length("a") == 17 and len(m.block_table("a", 0)) == 2
    m.reserve("a", 15); m.commit("a", 15)          # fills the second page exactly
    assert len(m.block_table("a", 0)) == 2
    m.reserve("a", 1); m.commit("a", 1)            # the first token of a third page
    assert len(m.block_table("a", 0)) == 3
    table = m.block_table("a", 0)
    assert m.slot("a", 0, 0) == table[0] * 16 and m.slot("a", 0, 32) == table[2] * 16 and m.slot("a", 0, 31) == table[1] * 16 + 15
    m.check_invariants()


def test_out_of_pages_takes_nothing_and_close_gives_everything_back():
    m = manager(num_pages=4)
    m.open("a"); m.open("b")
    m.reserve("a", 40); m.commit("a", 40)          # 3 pages
    with pytest.raises(OutOfPages):
        m.reserve("b", 17)                         # needs 2, 1 free
    assert m.free_pages() == [1] and m.block_table("b", 0) == []
    assert m.can_reserve([("b", 16)]) and not m.can_reserve([("b", 16), ("a", 9)])
    m.check_invariants()
    m.close("a")
    assert m.free_pages() == [4]
    with pytest.raises(CacheError):
        m.close("a")                               # closed twice
    m.reserve("b", 64); m.commit("b", 64)
    m.check_invariants()


def test_pages_are_used_again():
    m = manager(num_pages=2)
    m.open("a"); m.reserve("a", 32); m.commit("a", 32)
    first = list(m.block_table("a", 0))
    m.close("a")
    m.open("b"); m.reserve("b", 20); m.commit("b", 20)
    assert set(m.block_table("b", 0)) == set(first)


def test_rollback_of_a_step_that_did_not_run():
    m = manager()
    m.open("a"); m.reserve("a", 10); m.commit("a", 10)
    m.reserve("a", 30)
    assert m.free_pages() == [5]
    m.rollback("a")
    assert m.free_pages() == [7] and m.length("a") == 10 and len(m.block_table("a", 0)) == 1
    m.check_invariants()


def test_request_slots_and_length_limit():
    m = manager(max_requests=2, max_length=40)
    m.open("a"); m.open("b")
    assert not m.can_open()
    with pytest.raises(OutOfPages):
        m.open("c")
    with pytest.raises(CacheError, match="already open"):
        m.open("a")
    with pytest.raises(CacheError, match="exceed"):
        m.reserve("a", 41)
    assert m.requests["a"].state_slot != m.requests["b"].state_slot
    m.close("a"); m.open("c")
    m.check_invariants()


def test_window_group_gives_back_pages_it_has_passed():
    m = manager(groups=(FULL, WINDOW), num_pages={"full": 16, "win": 5}, page_size=16)
    m.open("a")
    for _ in range(12):                             # 12 * 13 = 156 tokens, far more than 5 pages of 16
        m.reserve("a", 13); m.commit("a", 13)
        m.check_invariants()
    full, win = m.block_table("a", 0), m.block_table("a", 1)
    assert len(full) == len(win) == 10 and NO_PAGE not in full
    # the next query is at 156 and reads keys 117..156: blocks before 117 // 16 = 7 are gone
    assert [p == NO_PAGE for p in win] == [True] * 7 + [False] * 3
    assert m.free_pages() == [6, 2]
    with pytest.raises(CacheError, match="given back"):
        m.slot("a", 1, 50)
    m.close("a")
    assert m.free_pages() == [16, 5]


def test_window_group_runs_out_only_when_the_window_does_not_fit():
    m = manager(groups=(WINDOW,), num_pages={"win": 4}, page_size=16)
    m.open("a")
    m.reserve("a", 60); m.commit("a", 60)          # 4 pages; after it blocks before (60-39)//16 = 1 are free
    assert m.free_pages() == [1]
    with pytest.raises(OutOfPages):
        m.reserve("a", 40)                          # one portion that needs 3 new pages at once
    m.reserve("a", 16); m.commit("a", 16)
    m.check_invariants()


@pytest.mark.parametrize("seed", range(6))
def test_random_orders_keep_the_invariants(seed):
    rng = random.Random(seed)
    groups = (FULL, WINDOW) if seed % 2 else (FULL,)
    m = manager(groups=groups, num_pages={"full": 12, "win": 6}, page_size=16, max_requests=5, max_length=200)
    live, next_id = {}, 0
    for _ in range(600):
        action = rng.random()
        if action < 0.25 and m.can_open():
            m.open(next_id); live[next_id] = 0; next_id += 1
        elif action < 0.85 and live:
            r = rng.choice(list(live))
            n = rng.choice([1, 1, 1, 2, 5, 16, 17, 40])
            free_before = m.free_pages()
            try:
                m.reserve(r, n)
            except (OutOfPages, CacheError):
                assert m.free_pages() == free_before      # a refusal changes nothing
            else:
                if rng.random() < 0.1:
                    m.rollback(r)
                else:
                    m.commit(r, n); live[r] += n
                    assert m.length(r) == live[r]
        elif live:
            r = rng.choice(list(live))
            m.close(r); del live[r]
        m.check_invariants()
    for r in list(live):
        m.close(r)
    m.check_invariants()
    assert m.free_pages() == [p.num_pages for p in m.pools]


def test_state_slots_exist_even_without_state(tmp_path):
    # with a state need and a device the slot's tensor is cleared at admission
    import torch

    m = CacheManager([FULL], {0: StateNeed((3,), torch.float32)}, num_pages=2, page_size=16, max_requests=2,
                     dtype=torch.float32, device="cpu")
    m.open("a")
    slot = m.requests["a"].state_slot
    m.state[0][slot] += 5
    m.close("a"); m.open("b")
    assert m.requests["b"].state_slot == slot and (m.state[0][slot] == 0).all()
    assert m.k_pages[0].shape == (2, 2, 16, 16) and m.v_pages[1].shape == (2, 2, 16, 16)


def test_capacity_from_memory():
    from mini_llm_amd.engine.loading import cache_bytes_per_token, tokens_for_memory

    small = [CacheGroupSpec("full", tuple(range(12)), 12, 64, None)]
    assert cache_bytes_per_token(small, 2) == 36864 and cache_bytes_per_token(small, 4) == 73728   # GPT-2 small: 73,728 bytes a token in 32-bit
    assert tokens_for_memory(small, 4, 4.5, 64) == 65536                     # 64 contexts of 1,024 tokens are 4.5 GiB
    two = small + [CacheGroupSpec("window", (12, 13), 2, 32, 100)]
    assert cache_bytes_per_token(two, 2) == 36864 + 2 * 2 * 2 * 32 * 2
    assert tokens_for_memory(two, 2, 1.0, 128) % 128 == 0
    with pytest.raises(ValueError):
        tokens_for_memory(small, 4, 1e-6, 64)
    with pytest.raises(ValueError):
        tokens_for_memory([], 4, 1.0, 64)


def test_a_slot_says_whether_its_own_request_has_been_sampled():
    # the last-token slot keeps what its previous owner left: a new owner has no token there until a sampler says so
    from mini_llm_amd.cache import CacheManager
    from mini_llm_amd.models.base import CacheGroupSpec

    cache = CacheManager([CacheGroupSpec("full", (0,), 1, 16, None)], {}, num_pages=4, page_size=4, max_requests=1)
    cache.open("a")
    assert not cache.has_sampled_token("a")
    cache.note_sampled("a")
    assert cache.has_sampled_token("a")
    cache.close("a")
    cache.open("b")                      # the same slot
    assert not cache.has_sampled_token("b")
