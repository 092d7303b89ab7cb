"""The cache manager on the CPU: no page lost, held twice or freed twice, under random orders of
requests; tail reuse, all-or-nothing allocation, windows, groups, slots and block tables.
(In the spirit of crates/cuda-kernels/src/paged_kv.rs:1758-2354, written fresh.)"""
import random

import pytest

from arle_amd.cache import (FREED, CacheManager, NoFreeSlot, OutOfPages, PagedNeed, PageGroup,
                            PagePool, StateNeed)


def test_pool_hands_out_page_zero_first_and_refuses_double_free():
    pool = PagePool(4)
    assert pool.take(2) == [0, 1]
    pool.give_back([1])
    assert pool.take(1) == [1]  # LIFO: a freed page is reused first
    with pytest.raises(AssertionError):
        pool.give_back([3])       # never held
    pool.give_back([0])
    with pytest.raises(AssertionError):
        pool.give_back([0])       # freed twice
    with pytest.raises(OutOfPages):
        pool.take(4)
    assert pool.free_count == 3   # the refused request took nothing


def test_tail_page_is_filled_before_a_new_page_is_taken():
    g = PageGroup(num_pages=8, page_size=4)
    g.open("a")
    assert g.pages_needed("a", 5) == 2
    g.append("a", 5)
    assert g.pages_needed("a", 3) == 0 and g.pages_needed("a", 4) == 1
    g.append("a", 3)
    assert len(g.tables["a"].pages) == 2 and g.tables["a"].length == 8
    assert g.free_tokens() == 6 * 4
    g.append("a", 1)
    assert g.free_tokens() == 5 * 4 + 3  # partial tail counts as free room
    g.check()


def test_token_to_page_map_and_truncate():
    g = PageGroup(num_pages=8, page_size=16)
    g.open("a")
    g.append("a", 40)
    pages = g.tables["a"].pages
    assert [pages[p // 16] for p in (0, 15, 16, 39)] == [pages[0], pages[0], pages[1], pages[2]]
    g.truncate("a", 17)
    assert len(g.tables["a"].pages) == 2 and g.pool.free_count == 6
    g.check()


def test_window_pages_are_given_back_while_the_request_runs():
    g = PageGroup(num_pages=6, page_size=4, window=6)
    g.open("a")
    g.append("a", 9)          # keys 0..8; next query at >= 9 reads keys >= 4
    assert g.trim("a") == [0]
    assert g.tables["a"].pages[0] == FREED and g.pool.free_count == 4
    g.append("a", 1)          # length 10: dead keys 0..4 -> still only page 0
    assert g.trim("a") == []
    g.append("a", 3)          # length 13: dead keys 0..7 -> page 1 too
    assert g.trim("a") == [1]
    g.check()
    # a long request needs only about window/page_size pages at a time
    for _ in range(40):
        g.append("a", 1)
        g.trim("a")
        g.check()
    assert g.pool.num_pages - g.pool.free_count <= 3
    g.close("a")
    assert g.pool.free_count == 6


def test_manager_all_or_nothing_across_requests_and_groups():
    needs = [PagedNeed(2, 16), PagedNeed(2, 16, window=8), PagedNeed(2, 16), None]
    m = CacheManager(needs, page_size=4, num_pages=5, max_slots=3, max_request_tokens=64, readers={3: 0})
    assert len(m.groups) == 2          # full-attention layers 0 and 2 share pages; the windowed layer has its own
    m.admit("a"), m.admit("b")
    m.append([("a", 9)])               # 3 pages in each group
    with pytest.raises(OutOfPages):
        m.append([("a", 3), ("b", 9)])  # a needs 0 more, b needs 3: only 2 free
    assert m.length("a") == 9 and m.length("b") == 0 and m.free_pages() == [2, 2]
    assert m.can_append([("b", 8)]) and not m.can_append([("b", 9)])
    m.trim_windows("a")
    assert m.free_pages() == [2, 2]    # window 8, length 9: keys 0..1 dead, page 0 still holds 2, 3
    m.append([("a", 3)])
    m.trim_windows("a")
    assert m.free_pages() == [2, 3]    # only the windowed group gave a page back
    m.check()
    view = m.view(3)
    assert view.writes is False and m.view(0).writes is True and m.view(1).window == 8
    m.release("a")
    assert m.free_pages() == [5, 5]
    m.check()


def test_slots_and_state_needs():
    m = CacheManager([StateNeed((4, 2)), PagedNeed(1, 16)], page_size=8, num_pages=4, max_slots=2,
                     max_request_tokens=32)
    s0, s1 = m.admit("a"), m.admit("b")
    assert {s0, s1} == {0, 1}
    with pytest.raises(NoFreeSlot):
        m.admit("c")
    with pytest.raises(KeyError):
        m.admit("a")
    m.release("a")
    assert m.admit("c") == s0          # a slot is used again
    with pytest.raises(OutOfPages, match="longest request"):
        m.append([("c", 33)])
    m.check()


def test_block_table_mirror_follows_the_pages():
    m = CacheManager([PagedNeed(1, 16)], page_size=4, num_pages=8, max_slots=2, max_request_tokens=32)
    sa = m.admit("a")
    m.append([("a", 6)])
    sb = m.admit("b")
    m.append([("b", 3)])
    m.append([("a", 5)])
    assert list(m._tables_host[0][sa, :3]) == m.table_of("a")
    assert list(m._tables_host[0][sb, :1]) == m.table_of("b")
    assert set(m.table_of("a")).isdisjoint(m.table_of("b"))


@pytest.mark.parametrize("seed", range(8))
def test_random_orders_lose_nothing(seed):
    rng = random.Random(seed)
    window = rng.choice([None, 5, 13])
    m = CacheManager([PagedNeed(2, 16), PagedNeed(2, 16, window=window)], page_size=rng.choice([1, 4, 16]),
                     num_pages=rng.randint(4, 24), max_slots=4, max_request_tokens=200)
    live, n_id = [], 0
    for _ in range(600):
        op = rng.random()
        if op < 0.2 and m.free_slot_count:
            key = f"r{n_id}"
            n_id += 1
            m.admit(key)
            live.append(key)
        elif op < 0.75 and live:
            batch = rng.sample(live, rng.randint(1, len(live)))
            appends = [(k, rng.randint(1, 12)) for k in batch]
            appends = [(k, n) for k, n in appends if m.length(k) + n <= 200]
            before = (m.free_pages(), {k: m.length(k) for k in live})
            if not appends:
                continue
            try:
                m.append(appends)
                for k, _ in appends:
                    m.trim_windows(k)
            except OutOfPages:
                assert (m.free_pages(), {k: m.length(k) for k in live}) == before
        elif op < 0.85 and live:
            k = rng.choice(live)
            m.truncate(k, rng.randint(0, m.length(k)))
        elif live:
            k = live.pop(rng.randrange(len(live)))
            m.release(k)
        m.check()
    for k in live:
        m.release(k)
    m.check()
    assert m.free_pages() == [g.pool.num_pages for g in m.groups]


def test_bytes_per_token_and_the_pool_sized_from_memory():
    # infer/src/model/qwen3/forward.rs:777-783: 2 (K+V) * layers * kv heads * head_dim * 2 bytes;
    # Qwen3-4B: 2 * 36 * 8 * 128 * 2 = 147,456
    import torch

    import arle_amd.models  # noqa: F401
    from arle_amd.cache import PAGE, PageTensor, cache_bytes_per_token, pages_for_memory, state_bytes_per_slot
    from arle_amd.config import Qwen3Config
    from arle_amd.models import declared_cache_needs, kv_cache_bytes_per_token
    from arle_amd.models.qwen3 import qwen3_spec

    cfg = Qwen3Config.from_dict(dict(num_hidden_layers=36, hidden_size=2560, num_attention_heads=32,
                                     num_key_value_heads=8, head_dim=128, intermediate_size=9728, vocab_size=151936,
                                     rope_theta=1e6, rms_norm_eps=1e-6, tie_word_embeddings=True,
                                     max_position_embeddings=40960))
    spec = qwen3_spec(cfg)
    assert kv_cache_bytes_per_token(spec, torch.bfloat16) == 147456
    assert kv_cache_bytes_per_token(spec, torch.float32) == 294912
    needs = declared_cache_needs(spec)
    assert len(needs) == 36 and needs[0] == PagedNeed(8, 128)
    # a need with tensors of its own: one compressed vector of 72 per token in float16, and an index in int8
    latent = PagedNeed(tensors=(PageTensor("latent", (PAGE, 72), torch.float16), PageTensor("tag", (PAGE,), torch.int8)))
    assert latent.bytes_per_token(torch.bfloat16) == 72 * 2 + 1
    assert cache_bytes_per_token([latent, None, PagedNeed(2, 16), StateNeed((4, 4))], torch.bfloat16) == 145 + 2 * 2 * 16 * 2
    assert state_bytes_per_slot([StateNeed((4, 4)), StateNeed((3,), torch.bfloat16), latent]) == 64 + 6
    with pytest.raises(ValueError, match="PAGE exactly once"):
        PagedNeed(tensors=(PageTensor("x", (4, 4)),)).bytes_per_token(torch.float32)
    # infer/src/scheduler/cuda/core/construction.rs:131-203: free - headroom, headroom = (1 - fraction) * total
    gib = 1 << 30
    page = 147456 * 16
    assert pages_for_memory(200 * gib, 288 * gib, 0.85, page) == int((200 - 288 * 0.15) * gib) // page
    assert pages_for_memory(200 * gib, 288 * gib, 0.85, page, most_pages=1000) == 1000
    assert pages_for_memory(10 * gib, 288 * gib, 0.85, page) == 0          # less free than the headroom
    assert pages_for_memory(100 * gib, 288 * gib, 1.0, page, reserved_bytes=gib) == (99 * gib) // page
    with pytest.raises(ValueError):
        pages_for_memory(1, 1, 0.0, 1)


def test_a_group_with_tensors_of_its_own_keeps_its_bookkeeping():
    import torch

    from arle_amd.cache import PAGE, PageTensor

    latent = PagedNeed(tensors=(PageTensor("latent", (PAGE, 24), torch.float32),), window=None)
    m = CacheManager([latent, PagedNeed(1, 16), latent], page_size=4, num_pages=6, max_slots=2, max_request_tokens=16)
    assert len(m.groups) == 2                      # the two latent entries share pages and a block table
    m.admit("a")
    m.append([("a", 9)])
    assert m.free_pages() == [3, 3]
    view = m.view(2)
    assert set(view.pages) == {"latent"} and view.writes and m.view(1).pages.keys() == {"k", "v"}
    m.release("a")
    m.check()
    assert m.free_pages() == [6, 6]
