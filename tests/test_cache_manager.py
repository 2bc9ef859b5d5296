"""The cache manager's bookkeeping: no page lost, held twice or freed twice, under random orders. No GPU."""
import numpy as np
import pytest
import torch

from microllm_rocm_amd.cache import RELEASED, CacheManager, OutOfPages, PagePool
from microllm_rocm_amd.parts import PagedKVNeed, StateNeed

FULL = PagedKVNeed(kv_heads=2, head_dim=16, window=None)
WINDOW = PagedKVNeed(kv_heads=2, head_dim=16, window=24)


def manager(needs=(FULL, FULL), reads=None, page_size=16, num_pages=8, max_requests=4):
    reads = reads or [None] * len(needs)
    return CacheManager(list(needs), list(reads), page_size, num_pages, max_requests, device=None)


def test_pool_refuses_double_free_and_overdraw():
    pool = PagePool(4)
    pages = pool.take(3)
    assert pages == [0, 1, 2] and pool.num_free == 1 and pool.peak_held == 3
    with pytest.raises(OutOfPages):
        pool.take(2)
    assert pool.num_free == 1                      # nothing was taken by the failed call
    pool.give([1])
    with pytest.raises(ValueError, match="not held"):
        pool.give([1])
    with pytest.raises(ValueError, match="does not belong"):
        pool.give([9])
    assert pool.take(1) == [1]                     # the page given back last goes out first
    assert sorted(pool.held_pages()) == [0, 1, 2]


def test_pages_follow_token_counts_and_come_back():
    cache = manager()
    request = cache.open("a")
    cache.reserve(request, 17)
    assert cache.held_pages() == [2] and request.reserved == 17
    cache.commit(request, 17)
    assert request.num_tokens == 17 and cache.pages_needed(request, 15) == [0] and cache.pages_needed(request, 16) == [1]
    cache.reserve(request, 1)
    cache.commit(request, 1)
    assert cache.held_pages() == [2]
    other = cache.open("b")
    with pytest.raises(OutOfPages):
        cache.reserve(other, 16 * 7)               # 6 free pages
    assert cache.held_pages() == [2] and other.reserved == 0 and other.pages == [[]]
    cache.reserve(other, 16 * 6)
    assert cache.free_pages() == [0] and not cache.can_reserve(request, 15)
    cache.check()
    cache.close("b")
    assert cache.free_pages() == [6]
    with pytest.raises(KeyError):
        cache.close("b")
    with pytest.raises(KeyError):
        cache.open("a")
    cache.close("a")
    assert cache.free_pages() == [8] and cache.slots.num_free == 4
    cache.check()


def test_groups_by_need_and_window_release():
    cache = manager(needs=(FULL, WINDOW, WINDOW), num_pages=8)
    assert [group.need for group in cache.groups] == [FULL, WINDOW]
    assert [group.entries for group in cache.groups] == [[0], [1, 2]]
    request = cache.open("a")
    cache.reserve(request, 40)
    assert cache.held_pages() == [3, 3]
    cache.commit(request, 40)
    # the next query is at 40 and sees keys >= 17: block 0 (keys 0..15) has passed, block 1 (16..31) has not
    assert request.pages[1][0] == RELEASED and request.pages[1][1] != RELEASED
    assert cache.held_pages() == [3, 2]
    for _ in range(8):
        cache.reserve(request, 1)
        cache.commit(request, 1)
    # at 48 the oldest visible key is 25: still block 1
    assert cache.held_pages() == [3, 2]
    assert request.pages[1][1] != RELEASED
    cache.reserve(request, 8)
    cache.commit(request, 8)   # 56 tokens: oldest visible key is 33 -> block 1 has passed
    assert request.pages[1][1] == RELEASED and request.pages[0][1] != RELEASED
    cache.check()
    cache.close("a")
    assert cache.free_pages() == [8, 8]


def test_cancel_reservation_gives_back_only_what_it_took():
    cache = manager()
    request = cache.open("a")
    cache.reserve(request, 20)
    cache.commit(request, 20)
    cache.reserve(request, 30)
    assert cache.held_pages() == [4]
    cache.cancel_reservation(request)
    assert cache.held_pages() == [2] and request.reserved == 0 and request.num_tokens == 20
    with pytest.raises(ValueError):
        cache.commit(request, 1)
    cache.check()


def test_state_slots_and_shared_caches():
    state = StateNeed((3, 5), torch.float32)
    cache = CacheManager([FULL, state, None, FULL], [None, None, 0, None], 16, 4, 2, device=None)
    bindings = cache.bindings()
    assert bindings[2].group == bindings[0].group and not bindings[2].owned and bindings[0].owned
    assert bindings[1].need == state
    first, second = cache.open("a"), cache.open("b")
    assert {first.slot, second.slot} == {0, 1}
    with pytest.raises(OutOfPages, match="slots"):
        cache.open("c")
    cache.close("a")
    assert cache.open("c").slot == first.slot
    with pytest.raises(ValueError, match="has none"):
        CacheManager([None, None], [None, 0], 16, 4, 2, device=None)


def test_a_need_class_from_outside_is_grouped_sized_and_counted_like_the_package_s_own():
    """The manager asks a need how it lives (pages or slots), what a position costs and what to hand the mixer;
    it lists no kinds. Something that is no need at all is refused by name."""
    from dataclasses import dataclass
    from typing import Optional
    from microllm_rocm_amd.cache import Binding, CacheNeed

    @dataclass(frozen=True)
    class LatentNeed(CacheNeed):
        width: int
        window: Optional[int] = None
        paged = True

        def bytes_per_position(self, dtype):
            return 2 * self.width

        def bind(self, group, storage, owned):
            return LatentBinding(self, owned, group)

    @dataclass
    class LatentBinding(Binding):
        group: int = 0

    latent, windowed = LatentNeed(24), LatentNeed(24, window=20)
    cache = CacheManager([latent, FULL, windowed, latent, None], [None, None, None, None, 0], 16, 8, 2, device=None, max_portion=8)
    assert [type(group.need).__name__ for group in cache.groups] == ["LatentNeed", "PagedKVNeed", "LatentNeed"]
    assert cache.groups[0].entries == [0, 3] and cache.groups[2].need.window == 20
    assert cache.groups[2].pool.num_pages == 2 * 3, "a windowed group of any payload is sized by its window"
    bindings = cache.bindings()
    assert isinstance(bindings[0], LatentBinding) and bindings[3].group == bindings[0].group
    assert bindings[4].group == bindings[0].group and not bindings[4].owned
    assert cache.bytes_per_page(cache.groups[0]) == 2 * 16 * 48 and not cache.has_state
    request = cache.open("a")
    cache.reserve(request, 40)
    cache.commit(request, 40)
    assert cache.held_pages() == [3, 3, 2], "the window has passed the first page of its group"
    cache.close("a")
    cache.check()
    with pytest.raises(TypeError, match="unknown cache need"):
        CacheManager([("keys", 4)], [None], 16, 8, 2, device=None)


def test_exact_byte_accounting():
    # the style of tests/inference/scheduler_test.cpp:419-422: bytes are an exact formula of the sizes
    cache = manager(needs=(FULL, FULL, WINDOW), num_pages=8)
    assert cache.allocated_bytes() == 2 * 2 * 2 * 16 * 16 * 4 * 8 + 2 * 1 * 2 * 16 * 16 * 4 * 8
    request = cache.open("a")
    cache.reserve(request, 33)
    assert cache.active_bytes() == (2 * 2 + 2 * 1) * 2 * 16 * 16 * 4 * 3


@pytest.mark.parametrize("seed", range(6))
def test_random_orders_never_lose_a_page(seed):
    rng = np.random.default_rng(seed)
    cache = manager(needs=(FULL, WINDOW), num_pages=12, max_requests=4)
    live = {}
    next_id = 0
    for _ in range(600):
        action = rng.integers(0, 10)
        if action < 2 and len(live) < 4:
            live[next_id] = cache.open(next_id)
            next_id += 1
        elif action < 8 and live:
            key = list(live)[rng.integers(0, len(live))]
            request = live[key]
            count = int(rng.integers(1, 40))
            before = (cache.free_pages(), [list(p) for p in request.pages], request.reserved)
            try:
                cache.reserve(request, count)
            except OutOfPages:
                assert (cache.free_pages(), [list(p) for p in request.pages], request.reserved) == before
                continue
            if rng.integers(0, 5) == 0:
                cache.cancel_reservation(request)
            else:
                cache.commit(request, count)
                held = sum(page != RELEASED for page in request.pages[0])
                assert held == cache.blocks_for(request.num_tokens)        # the full group holds ceil(len / 16)
                first_needed = max(0, request.num_tokens - 24 + 1) // 16
                assert all(page == RELEASED for page in request.pages[1][:first_needed])
                assert all(page != RELEASED for page in request.pages[1][first_needed:])
        elif live:
            key = list(live)[rng.integers(0, len(live))]
            cache.close(key)
            del live[key]
        cache.check()
    for key in list(live):
        cache.close(key)
    cache.check()
    assert cache.free_pages() == [12, 12] and cache.slots.num_free == 4


def test_a_group_with_a_window_sizes_its_own_pool_and_long_requests_fit_it():
    from microllm_rocm_amd.cache.manager import pages_of_group, window_blocks
    # window 24, portions of at most 16, pages of 16: a request never holds more than 4 blocks of the windowed group
    assert window_blocks(24, 16, 16) == 4
    assert pages_of_group(WINDOW, 1000, 16, 4, 16) == 16 and pages_of_group(FULL, 1000, 16, 4, 16) == 1000
    assert pages_of_group(WINDOW, 1000, 16, 4, None) == 1000 and pages_of_group(WINDOW, 10, 16, 4, 16) == 10
    cache = CacheManager([FULL, WINDOW], [None, None], 16, 128, 2, device=None, max_blocks=64, max_portion=16)
    assert [group.pool.num_pages for group in cache.groups] == [128, 8]
    assert cache.allocated_bytes() == (128 + 8) * 2 * 2 * 16 * 16 * 4
    # two requests of 500 tokens each, in portions of up to 16: the windowed pool of 8 pages is enough, and the
    # bound on what a request holds is never passed
    rng = np.random.default_rng(0)
    requests = [cache.open(name) for name in "ab"]
    lengths = [0, 0]
    most = 0
    while min(lengths) < 500:
        which = int(rng.integers(0, 2)) if max(lengths) < 900 else int(np.argmin(lengths))
        count = int(rng.integers(1, 17))
        cache.reserve(requests[which], count)
        most = max(most, max(sum(page != RELEASED for page in request.pages[1]) for request in requests))
        cache.commit(requests[which], count)
        lengths[which] += count
        if rng.random() < 0.1:
            cache.check()
    assert most <= 4 and cache.most_blocks(cache.groups[1], 500, 16) == 4 and cache.most_blocks(cache.groups[0], 500, 16) == 32
    assert cache.most_blocks(cache.groups[1], 20, 16) == 2          # a short request never holds more than its length
    cache.check()
    # a portion longer than the pool was sized for is refused as a whole, nothing taken
    held = cache.held_pages()
    with pytest.raises(OutOfPages):
        cache.reserve(requests[0], 16 * 9)
    assert cache.held_pages() == held
    for name in "ab":
        cache.close(name)
    assert cache.free_pages() == [128, 8]
