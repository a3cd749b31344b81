"""The cache manager on the host: allocator vectors of the reference, windows, random orders."""
import random

import pytest

from tokenizer_amd.cache import (CacheManager, DoubleFree, NotFull, PageAllocator, Release, UnknownPage,
                                 pages_for_len, prefix_page_hash)
from tokenizer_amd.parts import CacheNeed

P = 16


# ---- vectors of qwen-infer/src/paged.rs:822-1226 -----------------------------------------------
def test_alloc_free_roundtrip():
    alloc = PageAllocator(8, P)
    ids = [alloc.alloc() for _ in range(8)]
    assert ids[0] == 0 and sorted(ids) == list(range(8))
    assert alloc.alloc() is None and alloc.free_count() == 0
    for page in ids:
        alloc.free_page(page)
    assert alloc.free_count() == 8
    assert alloc.alloc() == ids[-1]          # the page freed last is handed out next
    one = PageAllocator(8, P)
    popped = [one.alloc() for _ in range(8)]
    batched = PageAllocator(8, P)
    assert batched.alloc_n(8) == popped
    assert batched.alloc_n(1) is None and batched.free_count() == 0


def test_no_double_free():
    alloc = PageAllocator(2, P)
    page = alloc.alloc()
    alloc.free_page(page)
    with pytest.raises(DoubleFree):
        alloc.free_page(page)
    assert alloc.free_count() == 2          # the refused free pushed nothing
    assert alloc.alloc() == page
    assert alloc.alloc() != page
    assert alloc.alloc() is None
    with pytest.raises(UnknownPage):
        alloc.free_page(9)


def test_refused_alloc_n_pops_nothing():
    alloc = PageAllocator(2, P)
    assert alloc.alloc_n(3) is None
    assert alloc.free_count() == 2
    assert alloc.alloc() is not None and alloc.alloc() is not None
    assert alloc.alloc() is None and alloc.alloc_n(1) is None


def test_fragmentation_is_bounded():
    lengths = [1, 15, 16, 17, 31, 32, 33, 63, 64, 100, 127, 128, 200, 255, 256]
    alloc = PageAllocator(10_000, P)
    held, waste = [], 0
    for length in lengths:
        pages = pages_for_len(length, P)
        gap = pages * P - length
        assert gap < P
        waste += gap
        held.append(alloc.alloc_n(pages))
    assert waste < P * len(lengths)
    freed = 0
    for index, ids in enumerate(held):
        if index % 2 == 0:
            freed += len(ids)
            for page in ids:
                alloc.free_page(page)
            ids.clear()
    again = alloc.alloc_n(freed)
    assert len(again) == freed
    for page in again + [p for ids in held for p in ids]:
        alloc.free_page(page)
    assert alloc.free_count() == alloc.capacity()


def test_bytes_per_token_and_the_51_sequences():
    # paged.rs:940-1011 and BENCHMARKS.md:280-291: 24 layers, 2 kv heads, head 64, float32.
    per_token = 24 * 2 * 2 * 64 * 4
    assert per_token == 24_576
    lengths = [8, 16, 17, 24, 31, 32, 40, 48, 63, 64, 80, 96, 100, 127, 128, 160, 200, 255]
    used, seqs = 0, []
    while True:
        length = lengths[len(seqs) % len(lengths)]
        if used + pages_for_len(length, P) > 256:
            break
        used += pages_for_len(length, P)
        seqs.append(length)
    assert len(seqs) == 51
    assert sum(seqs) * per_token == 94_666_752 and used * P * per_token == 99_090_432
    # The pool that holds exactly those pages has that many bytes in float32 and half of them in bfloat16.
    import torch
    from tokenizer_amd.cache import CacheManager, CachePools
    needs = [CacheNeed("full", 2, 64)] * 24
    manager = CacheManager(needs, num_pages=used, page_size=P, max_requests=4)
    assert CachePools(manager, needs, torch.float32, "cpu").bytes() == 99_090_432
    assert CachePools(manager, needs, torch.bfloat16, "cpu").bytes() * 2 == 99_090_432


def test_shared_prefix_uses_fewer_pages_than_two_copies():
    prompt = [3] * 32
    alloc = PageAllocator(8, P)
    first = alloc.alloc_n(2)
    alloc.publish_prompt_pages(prompt, first)
    shared = alloc.take_shared_prefix(prompt)
    assert len(shared) == 2 and alloc.live_count() == 2
    assert alloc.refcount(first[0]) == 2 and alloc.refcount(first[1]) == 2 and alloc.peak_live == 2
    for page in first + shared:
        alloc.free_page(page)
    assert alloc.all_refcounts_zero() and alloc.cached_count() == 2
    alloc.reclaim_cached()
    assert alloc.free_count() == alloc.capacity()


def test_hash_collision_does_not_share():
    alloc = PageAllocator(8, P)
    page, other_page = alloc.alloc(), alloc.alloc()
    stored, other, child = (1,) * P, (2,) * P, (3,) * P
    assert alloc._publish_at(7, 0, None, stored, page)
    assert not alloc._publish_at(7, 0, None, other, other_page)
    assert alloc._find_at(7, 0, None, other) is None
    assert alloc._find_at(7, 0, None, stored) == page
    child_page = alloc.alloc()
    assert alloc._publish_at(99, 7, page, child, child_page)
    decoy = alloc.alloc()
    assert alloc._find_at(99, 7, decoy, child) is None      # not shared under another parent page
    assert alloc._find_at(99, 7, page, child) == child_page
    assert alloc.take_shared_prefix(list(other) + list(child)) == []
    h0 = prefix_page_hash(0, stored)
    prompt = [1] * (3 * P)
    owned = alloc.alloc_n(3)
    assert alloc._publish_at(h0, 0, None, other, other_page)
    alloc.publish_prompt_pages(prompt, owned)
    assert alloc.find_full_page(h0, owned[0], prompt[P:2 * P]) is None


def test_divergence_inside_a_page_shares_only_earlier_pages():
    left = [4] * 48
    right = list(left)
    right[20] = 9
    alloc = PageAllocator(8, P)
    pages = alloc.alloc_n(3)
    alloc.publish_prompt_pages(left, pages)
    assert alloc.take_shared_prefix(right) == [pages[0]]
    assert [alloc.refcount(p) for p in pages] == [2, 1, 1]


def test_extension_hits_the_shorter_prompts_last_full_page():
    short = [4] * (2 * P)
    long = short + [7] * P
    alloc = PageAllocator(8, P)
    first = alloc.alloc_n(2)
    alloc.publish_prompt_pages(short, first)
    assert alloc.take_shared_prefix(short[:-1]) == [first[0]]
    assert alloc.take_shared_prefix(long[:-1]) == [first[0], first[1]]


def test_one_sharer_leaving_keeps_the_page_and_eviction_order():
    prompt = [8] * 32
    alloc = PageAllocator(4, P)
    pages = alloc.alloc_n(2)
    alloc.publish_prompt_pages(prompt, pages)
    shared = alloc.take_shared_prefix(prompt)
    assert alloc.free_page(pages[0]) == Release.SHARED and alloc.free_page(pages[1]) == Release.SHARED
    assert alloc.refcount(shared[0]) == 1 and alloc.live_count() == 2
    one = PageAllocator(1, P)
    page = one.alloc()
    one.publish_full_page(0, [5] * 16, page)
    with pytest.raises(NotFull):
        one.publish_full_page(0, [5] * 15, page)
    assert one.free_page(page) == Release.CACHED
    assert one.available() == 1 and one.free_count() == 0
    assert one.alloc() is not None                       # evicted before None
    assert one.find_full_page(0, None, [5] * 16) is None and one.cached_count() == 0


def test_hash_chain_formula():
    # paged.rs:93-100: FNV offset xor parent, then xor token, times prime, wrapping.
    value = 0xCBF29CE484222325 ^ 5
    for token in (1, 2):
        value = ((value ^ token) * 0x100000001B3) % (1 << 64)
    assert prefix_page_hash(5, [1, 2]) == value
    assert prefix_page_hash(0, [1, 2]) != prefix_page_hash(0, [2, 1])


# ---- the manager ---------------------------------------------------------------------------------
FULL = CacheNeed("full", 2, 16)
WIN = CacheNeed("window", 2, 16, window=21)
NONE = CacheNeed("none", state_shape=(4,))


def test_groups_follow_the_needs():
    manager = CacheManager([FULL, WIN, FULL, NONE, WIN], num_pages=8, page_size=P, max_requests=2)
    assert manager.group_of_layer == [0, 1, 0, None, 1]
    assert [g.layers for g in manager.groups] == [[0, 2], [1, 4]]
    assert manager.state_layers == [3]
    assert not CacheManager([FULL, WIN], 8, P, 2, prefix_cache=True).prefix_cache
    assert CacheManager([FULL, FULL], 8, P, 2, prefix_cache=True).prefix_cache


def test_no_prefix_sharing_beside_state_of_fixed_size():
    """A layer that keeps state in the request's slot has seen every token; a request that attached a shared
    prefix would skip those tokens, so sharing is off whatever was asked for."""
    manager = CacheManager([NONE, FULL], 8, P, 2, prefix_cache=True)
    assert not manager.prefix_cache
    prompt = list(range(40))
    manager.add_request(1)
    manager.reserve(1, 40), manager.advance(1, 40), manager.publish(1, prompt)
    manager.add_request(2)
    assert manager.attach_shared_prefix(2, prompt + [7]) == 0 and manager.seq_len(2) == 0
    state_and_pages = CacheNeed("full", 2, 16, state_shape=(3,))
    assert not CacheManager([state_and_pages, FULL], 8, P, 2, prefix_cache=True).prefix_cache


def test_a_kind_of_cache_is_a_rule_for_what_is_kept():
    """Another kind registers how far behind a query its keys are read; the bookkeeping needs nothing else."""
    from tokenizer_amd.cache import manager as manager_module
    manager_module.CACHE_KINDS["twice_the_window"] = lambda need: 2 * need.window
    try:
        manager = CacheManager([CacheNeed("twice_the_window", 2, 16, window=10), FULL], 16, P, 1)
        assert manager.group_of_layer == [0, 1]
        manager.add_request("a")
        manager.reserve("a", 100), manager.advance("a", 100)
        assert manager.first_needed_position(0, 100) == 80 and manager.first_needed_position(1, 100) == 0
        assert [p >= 0 for p in manager.table("a", 0)] == [False] * 5 + [True] * 2     # positions below 80 are gone
        manager.release("a")
        manager.check_invariants()
    finally:
        del manager_module.CACHE_KINDS["twice_the_window"]
    with pytest.raises(ValueError, match="unknown cache kind"):
        CacheManager([CacheNeed("twice_the_window", 2, 16, window=10)], 16, P, 1)
    with pytest.raises(ValueError, match="needs a window"):
        CacheManager([CacheNeed("window", 2, 16)], 16, P, 1)


def test_reserve_is_all_or_nothing_and_release_returns_everything():
    manager = CacheManager([FULL, WIN], num_pages=4, page_size=P, max_requests=2)
    manager.add_request("a")
    assert manager.reserve("a", 40) and [len(t) for t in manager.requests["a"].tables] == [3, 3]
    manager.add_request("b")
    assert not manager.reserve("b", 17)                   # two pages wanted, one left in each group
    assert manager.requests["b"].tables == [[], []]
    assert manager.reserve("b", 16)
    with pytest.raises(Exception):
        manager.add_request("c")                          # no slot left
    manager.release("a")
    manager.release("b")
    manager.check_invariants()
    assert all(g.allocator.free_count() == 4 for g in manager.groups)
    assert manager.free_slot_count() == 2


def test_window_group_gives_pages_back_behind_the_window():
    manager = CacheManager([FULL, WIN], num_pages=16, page_size=P, max_requests=1)
    manager.add_request("a")
    manager.reserve("a", 100)
    manager.advance("a", 100)
    full, win = manager.requests["a"].tables
    assert all(p >= 0 for p in full)
    # The next query is at position 100 and reads keys from 79 on: pages 0..3 (positions < 64) are gone,
    # page 4 (64..79) still holds position 79.
    assert [p >= 0 for p in win] == [False] * 4 + [True] * 3
    assert manager.groups[1].allocator.live_count() == 3 and manager.groups[0].allocator.live_count() == 7
    manager.reserve("a", 101)
    manager.advance("a", 101)
    assert [p >= 0 for p in manager.requests["a"].tables[1]] == [False] * 5 + [True] * 2
    manager.check_invariants()
    manager.release("a")
    manager.check_invariants()


def test_prefix_sharing_through_the_manager():
    manager = CacheManager([FULL, FULL], num_pages=8, page_size=P, max_requests=3, prefix_cache=True)
    prompt = list(range(40))
    manager.add_request(1)
    assert manager.attach_shared_prefix(1, prompt) == 0
    manager.reserve(1, 40)
    manager.advance(1, 40)
    manager.publish(1, prompt)
    manager.add_request(2)
    assert manager.attach_shared_prefix(2, prompt + [99] * 5) == 32
    assert manager.table(2, 0) == manager.table(1, 0)[:2]
    assert manager.seq_len(2) == 32
    manager.add_request(3)
    assert manager.attach_shared_prefix(3, prompt[:32]) == 16     # the page of the last token stays private
    manager.check_invariants()
    for rid in (1, 2, 3):
        manager.release(rid)
    manager.check_invariants()
    assert manager.groups[0].allocator.cached_count() == 2 and manager.groups[0].allocator.all_refcounts_zero()


@pytest.mark.parametrize("seed", range(6))
def test_random_orders_lose_nothing(seed):
    rng = random.Random(seed)
    needs = [FULL, WIN, FULL] if seed % 2 else [FULL, FULL]
    manager = CacheManager(needs, num_pages=24, page_size=P, max_requests=4, prefix_cache=bool(seed % 3))
    live, next_id = {}, 0
    common = [rng.randrange(50) for _ in range(48)]
    for _ in range(600):
        action = rng.random()
        if action < 0.25 and manager.free_slot_count():
            tokens = (common[:rng.choice([0, 16, 32, 48])] + [rng.randrange(50) for _ in range(rng.randrange(1, 40))])
            manager.add_request(next_id)
            shared = manager.attach_shared_prefix(next_id, tokens)
            assert shared % P == 0 and shared < len(tokens)
            live[next_id] = tokens
            next_id += 1
        elif action < 0.8 and live:
            rid = rng.choice(list(live))
            tokens = live[rid]
            have = manager.seq_len(rid)
            grow = rng.randrange(1, 30)
            if have + grow > len(tokens):
                tokens.extend(rng.randrange(50) for _ in range(have + grow - len(tokens)))
            before = [list(t) for t in manager.requests[rid].tables]
            if manager.reserve(rid, have + grow):
                manager.advance(rid, have + grow)
                manager.publish(rid, tokens)
            else:
                assert [list(t) for t in manager.requests[rid].tables] == before
        elif live:
            rid = rng.choice(list(live))
            manager.release(rid)
            del live[rid]
        manager.check_invariants()
    for rid in list(live):
        manager.release(rid)
    manager.check_invariants()
    for group in manager.groups:
        assert group.allocator.all_refcounts_zero()
        group.allocator.reclaim_cached()
        assert group.allocator.free_count() == group.allocator.capacity()
    with pytest.raises(KeyError):
        manager.release(0)


def test_a_pool_the_kernels_cannot_address_is_refused_when_it_is_made():
    """The attention kernels count a layer's key elements with 32 bits: a pool beyond that is refused with the
    number of pages that would fit, before anything is allocated."""
    import torch
    from tokenizer_amd.cache.pools import CachePools
    need = CacheNeed("full", 2, 64)                      # 2 kv heads of 64: 2,048 elements a page of 16
    fits = 2 ** 31 // 2048 - 1
    CachePools(CacheManager([need], num_pages=fits, page_size=P, max_requests=1), [need], torch.bfloat16, "meta")
    with pytest.raises(ValueError, match=f"at most {fits} pages"):
        CachePools(CacheManager([need], num_pages=fits + 1, page_size=P, max_requests=1), [need], torch.bfloat16, "meta")
