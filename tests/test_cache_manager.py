"""Page pool, block tables, windows and state slots of the cache manager (host side only, no GPU)."""

import random

import pytest
import torch

from somi_inference_amd.cache import RELEASED, CacheError, CacheManager, OutOfPages, PagePool
from somi_inference_amd.engine import StepEntry, build_step
from somi_inference_amd.parts import PAGE, FixedStateSpec, PagedKVSpec, PagedSpec, PageTensor


def manager(num_blocks=20, block_size=4, needs=None, max_requests=8):
    needs = needs if needs is not None else [PagedKVSpec(2, 16), PagedKVSpec(2, 16)]
    return CacheManager(needs, block_size=block_size, num_blocks=num_blocks, max_requests=max_requests,
                        dtype=torch.float32, device="cpu", allocate_tensors=False)


def test_pool_reuses_freed_pages_first_and_counts():
    # reference: free stack popped from the end (core/paged_attention.py:27-45)
    pool = PagePool(4)
    a, b = pool.allocate(), pool.allocate()
    assert (a, b) == (3, 2) and pool.num_free == 2
    pool.release(a)
    assert pool.allocate() == a
    pool.allocate(), pool.allocate()
    with pytest.raises(OutOfPages):
        pool.allocate()


def test_pool_refuses_double_free_and_unknown_pages():
    pool = PagePool(2)
    page = pool.allocate()
    pool.release(page)
    with pytest.raises(CacheError):
        pool.release(page)
    with pytest.raises(CacheError):
        pool.release(7)


def test_five_tokens_in_pages_of_four_take_two_pages():
    # /root/reference/tests/core/test_paged_attention.py:141-166
    m = manager()
    m.register(0)
    m.reserve(0, 5)
    assert len(m.page_list(0, 0)) == 2 and m.num_tokens(0) == 0      # counted only at commit (reference :294-296)
    m.commit(0, 5)
    assert m.num_tokens(0) == 5
    m.reserve(0, 3)
    assert len(m.page_list(0, 0)) == 2                                 # positions 5..7 still fit page 1
    m.commit(0, 3)
    m.reserve(0, 1)
    assert len(m.page_list(0, 0)) == 3
    m.free(0)
    assert m.free_pages() == [20]
    m.check_invariants()


def test_duplicate_and_unknown_requests():
    m = manager()
    m.register("a")
    with pytest.raises(CacheError, match="already registered"):       # reference :150-154
        m.register("a")
    with pytest.raises(CacheError, match="not registered"):
        m.reserve("b", 1)
    m.free("a")
    with pytest.raises(CacheError, match="not registered"):
        m.free("a")


def test_slots_follow_pages_and_positions():
    # reference: a token lands in page[pos // bs] at slot pos % bs, from the un-advanced base
    # (/root/reference/tests/core/test_kv_cache_manager_write.py:36-132)
    m = manager(block_size=4)
    m.register(0)
    m.reserve(0, 6)
    pages = m.page_list(0, 0)
    assert m.slots(0, 0, 0, 6) == [pages[0] * 4 + i for i in range(4)] + [pages[1] * 4, pages[1] * 4 + 1]
    m.commit(0, 3)                    # as after a first portion of 3
    assert m.slots(0, 0, 3, 2) == [pages[0] * 4 + 3, pages[1] * 4]


def test_reserve_is_all_or_nothing():
    m = manager(num_blocks=3, block_size=4)
    m.register(0)
    m.register(1)
    m.reserve(0, 8)
    assert not m.can_reserve([(1, 5)]) and m.can_reserve([(1, 4)])
    with pytest.raises(OutOfPages):
        m.reserve(1, 5)
    assert m.page_list(0, 1) == [] and m.free_pages() == [1]
    m.check_invariants()


def test_window_group_has_its_own_pages_and_returns_passed_ones():
    needs = [PagedKVSpec(2, 16), PagedKVSpec(2, 16, window=6), PagedKVSpec(2, 16, window=6)]
    m = manager(num_blocks=10, block_size=4, needs=needs)
    assert len(m.groups) == 2 and m.groups[1].window == 6 and m.groups[1].runs == [1, 2]
    assert m.layer_caches[0].group == 0 and m.layer_caches[1].group == 1
    m.register(0)
    m.reserve(0, 13)
    m.commit(0, 13)
    # next token is at 13 and sees keys from 13 - 6 + 1 = 8: pages 0 and 1 (positions 0..7) are done
    assert m.page_list(1, 0)[:2] == [RELEASED, RELEASED] and RELEASED not in m.page_list(1, 0)[2:]
    assert RELEASED not in m.page_list(0, 0)
    assert m.free_pages() == [6, 8]
    with pytest.raises(CacheError, match="released"):
        m.slots(1, 0, 7, 1)
    m.check_invariants()
    m.free(0)
    assert m.free_pages() == [10, 10]


def test_state_slots_and_cache_sharing_runs():
    needs = [FixedStateSpec((3,)), PagedKVSpec(1, 8), 1, None]
    m = CacheManager(needs, block_size=4, num_blocks=4, max_requests=2, dtype=torch.float32, device="cpu")
    assert m.layer_caches[3] is None
    assert m.layer_caches[2].k is m.layer_caches[1].k and m.layer_caches[2].writes is False
    assert m.layer_caches[0].state.shape == (2 + 1, 3)         # a row per request and the one padding entries use
    assert m.padding_state_slot == 2
    m.register("a")
    m.layer_caches[0].state[m.state_slot("a")] = 5.0
    m.register("b")
    assert m.state_slot("a") != m.state_slot("b")
    with pytest.raises(CacheError, match="slots"):
        m.register("c")
    m.free("a")
    m.register("c")                                   # the slot is used again, and zeroed
    assert float(m.layer_caches[0].state[m.state_slot("c")].abs().sum()) == 0.0
    m.check_invariants()


@pytest.mark.parametrize("seed", range(6))
def test_random_orders_never_lose_hold_twice_or_free_twice(seed):
    rng = random.Random(seed)
    latent = (PageTensor("latent", (PAGE, 6)),)
    needs = [PagedKVSpec(1, 8), PagedKVSpec(1, 8, window=5), PagedSpec(latent, page_size=3),
             PagedSpec(latent, window=7, page_size=6)]
    m = manager(num_blocks=12, block_size=4, needs=needs, max_requests=5)
    assert [g.pool.num_pages for g in m.groups] == [12, 12, 16, 8]
    live, next_id = {}, 0
    for _ in range(400):
        action = rng.random()
        if action < 0.25 and len(live) < 5:
            m.register(next_id)
            live[next_id] = 0
            next_id += 1
        elif action < 0.4 and live:
            rid = rng.choice(list(live))
            m.free(rid)
            del live[rid]
        elif live:
            rid = rng.choice(list(live))
            count = rng.choice([1, 1, 1, 2, 3, 7])
            if m.can_reserve([(rid, count)]):
                m.reserve(rid, count)
                m.commit(rid, count)
                live[rid] += count
                assert m.num_tokens(rid) == live[rid]
            else:
                before = m.free_pages()
                with pytest.raises(OutOfPages):
                    m.reserve(rid, count)
                assert m.free_pages() == before
        m.check_invariants()
    for rid in list(live):
        m.free(rid)
    assert m.free_pages() == [12, 12, 16, 8]


def test_step_arrays_for_a_mixed_batch():
    m = manager(num_blocks=8, block_size=4, needs=[PagedKVSpec(1, 8)])
    m.register("p")
    m.register("d")
    m.reserve("d", 5)
    m.commit("d", 5)
    entries = [StepEntry("p", [9, 8, 7, 6, 5, 4], [5]), StepEntry("d", [3], [0])]
    for e in entries:
        m.reserve(e.request_id, len(e.tokens))
    step = build_step(entries, m, torch.device("cpu"))
    assert step.num_tokens == 7 and step.num_entries == 2 and step.num_logit_rows == 2
    assert step.token_ids.tolist() == [9, 8, 7, 6, 5, 4, 3]
    assert step.positions.tolist() == [0, 1, 2, 3, 4, 5, 5]
    assert step.token_entry.tolist() == [0, 0, 0, 0, 0, 0, 1]
    assert step.entry_start.tolist() == [0, 6, 7] and step.context_lens.tolist() == [6, 6]
    assert step.logit_rows.tolist() == [5, 6]
    table = step.paged[0].block_table
    assert table.shape == (2, 2)
    assert table[0].tolist() == m.page_list(0, "p") and table[1].tolist() == m.page_list(0, "d")
    assert step.paged[0].slot_mapping.tolist() == m.slots(0, "p", 0, 6) + m.slots(0, "d", 5, 1)
    assert step.max_entry_len == 6 and step.max_context == 6
    # no portion is longer than 8 tokens: every token is listed for the kernel that attends token by token
    assert not step.splits
    with pytest.raises(KeyError, match="entry_split"):
        step.split(8)
    # the lists a mixer asks for by declaring a threshold: entries longer than it, tokens of the others
    cut = build_step(entries, m, torch.device("cpu"), entry_splits=(8, 4)).split(8)
    assert cut.long_entry_len.tolist() == [0, 0] and cut.short_tokens.tolist() == [0, 1, 2, 3, 4, 5, 6]
    assert (cut.num_long_tokens, cut.num_short_tokens) == (0, 7)
    cut = build_step(entries, m, torch.device("cpu"), entry_splits=(8, 4)).split(4)
    assert cut.long_entry_len.tolist() == [6, 0] and cut.short_tokens.tolist() == [6]
    assert (cut.num_long_tokens, cut.num_short_tokens) == (6, 1)
    assert all(t.dtype == torch.int32 for t in (step.token_ids, step.positions, table, step.logit_rows))


def test_rollback_gives_back_what_a_failed_step_reserved_and_nothing_else():
    cache = CacheManager([PagedKVSpec(1, 8), PagedKVSpec(1, 8, window=6)], block_size=4, num_blocks=8,
                         max_requests=2, dtype=torch.float32, device="cpu", allocate_tensors=False)
    cache.register("a")
    cache.reserve("a", 10)
    cache.commit("a", 10)                       # the window of 6 has passed page 0 of the second group
    held = cache.free_pages()
    cache.reserve("a", 7)                       # 17 tokens: two more pages in each group
    assert cache.free_pages() == [held[0] - 2, held[1] - 2]
    cache.rollback("a")
    assert cache.free_pages() == held and cache.num_tokens("a") == 10
    cache.check_invariants()
    cache.rollback("a")                         # nothing reserved: nothing happens
    assert cache.free_pages() == held
    cache.reserve("a", 1)
    cache.commit("a", 1)
    cache.free("a")
    assert cache.free_pages() == [8, 8]
    cache.check_invariants()


def test_a_group_stores_what_its_spec_lists_in_pages_of_its_own_size():
    latent = PagedSpec((PageTensor("latent", (PAGE, 6), torch.float32), PageTensor("gate", (2, PAGE))), page_size=3)
    needs = [PagedKVSpec(2, 8), latent, PagedKVSpec(2, 8, page_size=3), latent, 1]
    m = CacheManager(needs, block_size=4, num_blocks=6, max_requests=2, dtype=torch.bfloat16, device="cpu")
    # keys and values at the engine's page size; the latent group and the k/v layer that asks for pages of 3
    # share tables (same window, same page size) and hold the pool's 24 tokens in 8 pages
    assert [(g.window, g.page_size, g.pool.num_pages, g.runs) for g in m.groups] == [(None, 4, 6, [0]), (None, 3, 8, [1, 2, 3])]
    kv, lat, kv3, lat2, reader = m.layer_caches
    assert kv.k.shape == (6, 2, 4, 8) and kv.v.shape == (6, 2, 8, 4) and kv.page_size == 4
    assert lat.tensors["latent"].shape == (8, 3, 6) and lat.tensors["latent"].dtype == torch.float32
    assert lat.tensors["gate"].shape == (8, 2, 3) and lat.tensors["gate"].dtype == torch.bfloat16
    assert lat.k is None and lat.page_size == 3
    assert kv3.k.shape == (8, 2, 3, 8) and kv3.group == lat.group == 1
    assert lat2.tensors["latent"] is not lat.tensors["latent"]
    assert reader.tensors["latent"] is lat.tensors["latent"] and not reader.writes and reader.page_size == 3
    assert CacheManager.page_bytes(needs, 4, torch.bfloat16) == 4 * (2 * 2 * 8 * 2 + (6 * 4 + 2 * 2) + 2 * 2 * 8 * 2 + (6 * 4 + 2 * 2))
    m.register("r")
    assert m.pages_needed("r", 7) == [2, 3]
    m.reserve("r", 7)
    m.commit("r", 7)
    assert m.slots(0, "r", 3, 3) == [m.page_list(0, "r")[0] * 4 + 3, m.page_list(0, "r")[1] * 4, m.page_list(0, "r")[1] * 4 + 1]
    assert m.slots(1, "r", 2, 2) == [m.page_list(1, "r")[0] * 3 + 2, m.page_list(1, "r")[1] * 3]
    # one more page in group 0 would hold up to token 12, two more in group 1 up to token 15
    assert m.tokens_within("r", [1, 2]) == 5 and m.tokens_within("r", [0, 0]) == 1
    assert m.holds(24) and not m.holds(25)
    step = build_step([StepEntry("r", [1], [0])], _reserved(m, "r", 1), torch.device("cpu"))
    assert [view.page_size for view in step.paged] == [4, 3]
    assert step.paged[1].block_table.shape == (1, 3) and step.paged[0].block_table.shape == (1, 2)
    m.check_invariants()
    with pytest.raises(ValueError, match="holds no page"):
        manager(num_blocks=1, block_size=4, needs=[PagedSpec((PageTensor("x", (PAGE,)),), page_size=5)])
    with pytest.raises(ValueError, match="PAGE exactly once"):
        PageTensor("x", (3, 4))


def _reserved(m, request_id, count):
    m.reserve(request_id, count)
    return m
