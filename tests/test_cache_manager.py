"""The cache manager on the CPU: pages are never lost, held twice or freed twice."""

import random

import pytest

from clockwork_amd.cache import NO_PAGE, CacheManager, OutOfPages, PagePool, PrefixCache, plan_groups
from clockwork_amd.config.spec import KVPagesSpec, StateSpec

BS = 4


def manager(num_blocks=16, watermark=0.0, needs=None, max_num_seqs=8, block_size=BS):
    needs = needs if needs is not None else [KVPagesSpec(2, 16)] * 3
    return CacheManager(plan_groups(needs), block_size, num_blocks, max_num_seqs=max_num_seqs, watermark=watermark)


# ------------------------------------------------------------------ the pool
def test_pool_hands_out_ascending_then_reuses_last_freed_first():
    # clockwork/kvcache/block.py:17,35,56
    pool = PagePool(4, BS)
    assert [pool.take() for _ in range(4)] == [0, 1, 2, 3]
    with pytest.raises(OutOfPages):
        pool.take()
    pool.drop(1)
    pool.drop(3)
    assert pool.take() == 3 and pool.take() == 1


def test_pool_refuses_double_free_and_bad_ids():
    pool = PagePool(4, BS)
    page = pool.take()
    pool.drop(page)
    with pytest.raises(ValueError, match="has no holder"):
        pool.drop(page)
    with pytest.raises(ValueError, match="outside this pool"):
        pool.share(4)
    with pytest.raises(ValueError, match="one at a time"):
        pool.hold(pool.take(), 2)
    with pytest.raises(ValueError):
        PagePool(0, BS)


def test_take_many_is_all_or_nothing():
    pool = PagePool(4, BS)
    pool.take()
    with pytest.raises(OutOfPages):
        pool.take_many(4)
    assert pool.num_free == 3
    assert len(pool.take_many(3)) == 3


def test_private_copy_takes_the_new_page_before_letting_go():
    pool = PagePool(2, BS)
    page = pool.take()
    assert pool.private_copy(page) is None  # one holder: nothing to copy
    pool.share(page)
    other = pool.take()
    with pytest.raises(OutOfPages):
        pool.private_copy(page)
    assert pool.refcount(page) == 2  # untouched by the failure (tests/test_block_allocator.py)
    pool.drop(other)
    assert pool.private_copy(page) == (page, other)
    assert pool.refcount(page) == 1 and pool.refcount(other) == 1


def test_pool_fuzz_against_a_dict_model():
    rng = random.Random(0)
    pool = PagePool(12, BS)
    model: dict[int, int] = {}
    for _ in range(600):
        op = rng.choice(["take", "share", "drop", "cow"])
        if op == "take":
            if len(model) == 12:
                with pytest.raises(OutOfPages):
                    pool.take()
            else:
                page = pool.take()
                assert page not in model
                model[page] = 1
        elif model:
            page = rng.choice(sorted(model))
            if op == "share":
                pool.share(page)
                model[page] += 1
            elif op == "drop":
                pool.drop(page)
                model[page] -= 1
                if model[page] == 0:
                    del model[page]
            elif model[page] > 1 and len(model) < 12:
                src, dst = pool.private_copy(page)
                model[src] -= 1
                model[dst] = 1
        assert pool.num_free + len(model) == 12
        for page in range(12):
            assert pool.refcount(page) == model.get(page, 0)
        pool.audit()


# ------------------------------------------------------------------ groups
@pytest.mark.parametrize("seed", range(6))
def test_many_holds_at_once_equal_one_hold_after_the_other(seed):
    """The array form of a request's holds leaves the counts and the order of the free stack
    that a loop of single holds leaves, also when a page is named twice or is not in use."""
    rng = random.Random(seed)
    num_pages = rng.choice([12, 40, 97])
    fast, slow = PagePool(num_pages, 4), PagePool(num_pages, 4)
    for pool in (fast, slow):
        pool.take_many(num_pages - 3)
    for _ in range(60):
        in_use = [p for p in range(num_pages) if slow.refcount(p) > 0]
        step = rng.choice([1, -1])
        pages = rng.sample(in_use, rng.randint(0, len(in_use))) if in_use else []
        if pages and rng.random() < 0.15:
            pages.append(rng.choice(pages))  # the same page twice
        failed = []
        for pool, call in ((fast, lambda: fast.hold_many(pages, step)),
                           (slow, lambda: [slow.hold(page, step) for page in pages])):
            try:
                call()
                failed.append(None)
            except ValueError as err:
                failed.append(str(err))
        assert failed[0] == failed[1]
        if failed[0] is not None:  # a loop stops half way, the array form before it starts
            fast, slow = PagePool(num_pages, 4), PagePool(num_pages, 4)
            for pool in (fast, slow):
                pool.take_many(num_pages - 3)
            continue
        assert fast._holders.tolist() == slow._holders.tolist()
        assert fast._idle[: fast.num_free].tolist() == slow._idle[: slow.num_free].tolist()
        fast.audit()
        if slow.num_free > 4 and rng.random() < 0.5:
            n = rng.randint(1, slow.num_free)
            assert fast.take_many(n) == slow.take_many(n)
    with pytest.raises(ValueError, match="no holder"):
        free_page = PagePool(16, 4)
        held = free_page.take_many(10)
        free_page.drop(held[3])
        free_page.hold_many(held, -1)
    assert free_page.refcount(held[0]) == 1  # refused before anything changed
    with pytest.raises(ValueError, match="outside"):
        free_page.hold_many([0, 1, 2, 4, 5, 6, 7, 8, 99], 1)


def test_layers_with_the_same_need_share_a_group():
    needs = [KVPagesSpec(2, 16), KVPagesSpec(2, 16, window=8), KVPagesSpec(2, 16), None, StateSpec((4,)), KVPagesSpec(2, 16, window=8)]
    groups = plan_groups(needs)
    assert [(g.entries, g.window) for g in groups if g.is_kv] == [((0, 2), None), ((1, 5), 8)]
    assert [g.entries for g in groups if not g.is_kv] == [(4,)]
    with pytest.raises(TypeError):
        plan_groups(["pages"])


# ------------------------------------------------------------------ admission and growth
def test_admission_covers_the_request_with_ceil_div_pages():
    m = manager()
    rec = m.admit("a", total_len=9)
    assert rec.tables == [[0, 1, 2]]
    assert m.num_free_blocks() == 13
    with pytest.raises(ValueError, match="already holds"):
        m.admit("a", 4)


def test_watermark_exactly_at_and_below_the_threshold():
    # tests/test_block_manager.py:91-102: 16 pages, watermark 0.25 -> 4 must stay free
    m = manager(num_blocks=16, watermark=0.25)
    assert m.can_admit(12 * BS)
    assert not m.can_admit(12 * BS + 1)
    m.admit("a", 12 * BS)
    assert m.num_free_blocks() == 4
    # pages that come from the prefix cache cost nothing (tests/test_block_manager.py:105-115)
    m2 = manager(num_blocks=16, watermark=0.25)
    m2.pools[0].take_many(4)
    assert not m2.can_admit(9 * BS)
    assert m2.can_admit(9 * BS, prefix_blocks=4)


def test_growth_needs_a_page_only_at_a_page_edge():
    m = manager(num_blocks=3)
    m.admit("a", 7)  # 2 pages, one slot left in the second
    assert m.can_extend("a", 7, 8) and m.extend("a", 7, 8) == []
    assert m.block_table("a") == [0, 1]
    m.extend("a", 8, 9)
    assert m.block_table("a") == [0, 1, 2]
    m.admit_ok = m.can_extend("a", 12, 13)
    assert not m.admit_ok  # position 12 opens a fourth page and none is free
    with pytest.raises(OutOfPages):
        m.extend("a", 12, 13)
    assert m.block_table("a") == [0, 1, 2]  # state intact after the failure


def test_fork_shares_pages_and_a_write_under_a_shared_page_copies_it():
    m = manager(num_blocks=6)
    m.admit("parent", 6)
    m.fork("parent", "child")
    assert m.block_table("child") == m.block_table("parent") == [0, 1]
    assert m.pools[0].refcount(1) == 2
    copies = m.extend("child", 6, 7)  # position 6 lies in shared page 1
    assert copies == [(0, 1, 2)]
    assert m.block_table("child") == [0, 2] and m.block_table("parent") == [0, 1]
    assert m.extend("parent", 6, 7) == []  # the parent is the only holder now
    m.free("parent")
    m.free("child")
    assert m.num_free_blocks() == 6


def test_free_gives_everything_back_and_refuses_a_second_time():
    m = manager()
    m.admit("a", 10)
    m.free("a")
    assert m.num_free_blocks() == 16
    with pytest.raises(ValueError, match="double free"):
        m.free("a")


def test_slot_mapping_layout_and_range_errors():
    # tests/test_block_manager.py:270-281
    m = manager()
    m.pools[0].take_many(3)  # make the request's pages non-trivial: 3, 4
    m.admit("a", 6)
    assert m.slot_mapping("a", 0, 6) == [12, 13, 14, 15, 16, 17]
    assert m.slot_mapping("a", 3, 5) == [15, 16]
    with pytest.raises(ValueError, match="outside covered range"):
        m.slot_mapping("a", 0, 9)


# ------------------------------------------------------------------ windows
def test_a_windowed_group_gives_pages_back_while_the_request_runs():
    needs = [KVPagesSpec(1, 16), KVPagesSpec(1, 16, window=6)]
    m = manager(num_blocks=8, needs=needs)
    m.admit("a", total_len=30, portion_end=10)
    # the full group reserves the whole request, the windowed group only the first portion
    assert len(m.block_table("a", 0)) == 8 and len(m.block_table("a", 1)) == 3
    assert m.release_behind_window("a", 10) == 1  # next token (position 10) reads 5..10: page 0 is behind
    assert m.block_table("a", 1) == [NO_PAGE, 1, 2]
    m.extend("a", 10, 20)
    assert m.block_table("a", 1)[3:] == [0, 3]  # the page given back is used again
    assert m.release_behind_window("a", 20) == 2
    assert m.block_table("a", 1) == [NO_PAGE, NO_PAGE, NO_PAGE, 0, 3]
    with pytest.raises(ValueError, match="given back"):
        m.slot_mapping("a", 8, 12, group=1)
    assert m.slot_mapping("a", 16, 18, group=1) == [3 * BS + 0, 3 * BS + 1]
    m.free("a")
    assert [p.num_free for p in m.pools] == [8, 8]
    assert not m.supports_prefix_sharing


def test_window_group_pages_stay_bounded_over_a_long_request():
    m = manager(num_blocks=5, needs=[KVPagesSpec(1, 16, window=5)])
    m.admit("a", total_len=400, portion_end=3)
    at = 3
    while at < 400:
        m.release_behind_window("a", at)
        n = min(7, 400 - at)
        m.extend("a", at, at + n)
        at += n
        assert m.pools[0].num_free >= 1
    m.free("a")
    assert m.pools[0].num_free == 5


# ------------------------------------------------------------------ state slots
def test_state_slots_are_handed_out_and_returned():
    m = manager(needs=[KVPagesSpec(1, 16), StateSpec((8,))], max_num_seqs=2)
    a = m.admit("a", 4)
    b = m.admit("b", 4)
    assert {a.state_slot, b.state_slot} == {0, 1}
    assert not m.can_admit(4)
    with pytest.raises(OutOfPages, match="state slot"):
        m.admit("c", 4)
    m.free("a")
    assert m.admit("c", 4).state_slot == a.state_slot
    with pytest.raises(OutOfPages, match="state slot"):
        m.fork("b", "d")  # a fork needs a slot of its own: state is copied, never shared
    m.free("c")
    src, dst = m.fork("b", "d")
    assert src == b.state_slot and dst == m.state_slot("d") and dst != src
    assert not m.supports_prefix_sharing


def test_a_model_without_state_hands_out_no_slot():
    m = manager()
    assert m.admit("a", 4).state_slot == -1


# ------------------------------------------------------------------ random orders of requests
@pytest.mark.parametrize("seed", range(5))
def test_random_request_orders_never_lose_or_duplicate_a_page(seed):
    rng = random.Random(seed)
    needs = [KVPagesSpec(1, 16), KVPagesSpec(1, 16, window=9), StateSpec((2,))]
    m = manager(num_blocks=24, needs=needs, max_num_seqs=5)
    live: dict[str, list[int]] = {}  # id -> [length, total]
    serial = 0
    for _ in range(800):
        op = rng.random()
        if op < 0.25 and len(live) < 5:
            total = rng.randint(1, 40)
            first = rng.randint(1, total)
            if m.can_admit(total, first):
                sid = f"s{serial}"
                serial += 1
                m.admit(sid, total, first)
                m.extend(sid, 0, first)
                live[sid] = [first, total]
        elif op < 0.8 and live:
            sid = rng.choice(sorted(live))
            length, total = live[sid]
            m.release_behind_window(sid, length)
            n = rng.randint(1, 6)
            if m.can_extend(sid, length, length + n):
                m.extend(sid, length, length + n)
                live[sid][0] = length + n
                m.slot_mapping(sid, length, length + n, 0)
                m.slot_mapping(sid, length, length + n, 1)
        elif live:
            sid = rng.choice(sorted(live))
            m.free(sid)
            del live[sid]
        # every page is free or held by exactly the requests whose tables name it
        for g, pool in enumerate(m.pools):
            pool.audit()
            held: dict[int, int] = {}
            for sid in live:
                for page in m.block_table(sid, g):
                    if page != NO_PAGE:
                        held[page] = held.get(page, 0) + 1
            assert all(count == 1 for count in held.values()), "a page is held twice"
            assert pool.num_free + len(held) == 24, "a page was lost"
        slots = [m.state_slot(sid) for sid in live]
        assert len(set(slots)) == len(slots)
    for sid in list(live):
        m.free(sid)
    assert all(p.num_free == 24 for p in m.pools)


# ------------------------------------------------------------------ sizing the pools
def test_pages_that_fit_follows_the_reference_arithmetic_and_its_caps():
    import torch

    from clockwork_amd.cache.pools import page_bytes, pages_that_fit

    # 28 layers, block 16, 2 kv heads of 128, 2 bytes: 458,752 bytes a page
    # (configs/qwen2.5-1.5b-instruct-cuda.yaml:24-34)
    groups = plan_groups([KVPagesSpec(2, 128)] * 28)
    assert page_bytes(groups, 16, torch.bfloat16) == 458752
    assert page_bytes(groups, 16, torch.float32) == 2 * 458752
    free = 100 * 458752 + 17
    assert pages_that_fit(groups, 16, torch.bfloat16, free, 1.0, most=10 ** 9) == 100
    assert pages_that_fit(groups, 16, torch.bfloat16, free, 0.5, most=10 ** 9) == 50
    assert pages_that_fit(groups, 16, torch.bfloat16, free, 1.0, most=64) == 64
    with pytest.raises(RuntimeError, match="no room"):
        pages_that_fit(groups, 16, torch.bfloat16, 1000, 1.0, most=64)
    with pytest.raises(ValueError, match="memory_fraction"):
        pages_that_fit(groups, 16, torch.bfloat16, free, 0.0, most=64)
    # two groups (all keys / a window) each have a pool: a page number costs both
    two = plan_groups([KVPagesSpec(2, 16), KVPagesSpec(2, 16, window=8), KVPagesSpec(2, 16)])
    assert page_bytes(two, 4, torch.float32) == 3 * 2 * 4 * 2 * 16 * 4
    # a model without paged state needs no pages
    assert pages_that_fit(plan_groups([StateSpec((4,), "float32")]), 16, torch.float32, 10, 1.0, most=5) == 1


# ------------------------------------------------------------------ pages of a mixer's own rows
def test_a_mixer_may_keep_planes_of_its_own_in_pages():
    """Keys and values of one shape are one case; a mixer may cache one latent vector a token
    and no values, or planes of different widths. The manager pages them all alike, the pools
    size every plane from the spec."""
    import torch

    from clockwork_amd.cache.pools import CachePools, page_bytes
    from clockwork_amd.config.spec import PagedRowsSpec

    latent = PagedRowsSpec((("latent", (24,)),))
    uneven = PagedRowsSpec((("k", (2, 16)), ("v", (2, 8))), window=8)
    assert KVPagesSpec(2, 16).planes == (("k", (2, 16)), ("v", (2, 16)))
    assert latent.group_key() != PagedRowsSpec((("latent", (32,)),)).group_key()
    with pytest.raises(ValueError, match="names of their own"):
        PagedRowsSpec((("a", (4,)), ("a", (4,))))
    with pytest.raises(ValueError, match="row shape"):
        PagedRowsSpec((("a", ()),))
    groups = plan_groups([latent, KVPagesSpec(2, 16), latent, uneven, StateSpec((4,), "float32")])
    assert [(g.is_kv, g.window, g.entries) for g in groups] == [
        (True, None, (0, 2)), (True, None, (1,)), (True, 8, (3,)), (False, None, (4,))]
    # a page number costs: two entries of 24, one of 2 x 2 x 16, one of 2 x 16 + 2 x 8, times the page's tokens
    assert page_bytes(groups, 4, torch.float32) == 4 * 4 * (2 * 24 + 64 + 48)
    m = CacheManager(groups, block_size=4, num_blocks=6, max_num_seqs=2)
    m.admit("a", 9)
    assert [len(m.block_table("a", g)) for g in range(3)] == [3, 3, 3]
    m.free("a")
    assert all(p.num_free == 6 for p in m.pools)

    pools = CachePools(groups, 4, 6, 2, torch.float32, "cpu", fill=7.0)
    assert tuple(pools.kv[0].shape) == (2, 1, 6, 4, 24) and tuple(pools.kv[1].shape) == (1, 2, 6, 4, 2, 16)
    assert pools.kv[2] is None   # planes of different shapes have a tensor each
    assert {n: tuple(t.shape) for n, t in pools.planes[2].items()} == {"k": (1, 6, 4, 2, 16), "v": (1, 6, 4, 2, 8)}
    assert pools.kv_bytes_per_token() == 4 * (2 * 24 + 64 + 48)
    assert pools.bytes() == 6 * 4 * pools.kv_bytes_per_token() + 4 * 4 * 4
    cache = pools.entry_cache(2)     # the second entry of the latent group
    assert cache.group == 0 and cache.k is None and cache.v is None and tuple(cache.planes["latent"].shape) == (24, 24)
    cache.planes["latent"][5] = 1.0  # a view of the pool: page 1, token 1 of entry row 1
    assert float(pools.kv[0][1, 0, 1, 1].sum()) == 24.0 and float(pools.kv[0][0].sum()) == 7.0 * 6 * 4 * 24
    kv = pools.entry_cache(1)
    assert tuple(kv.k.shape) == tuple(kv.v.shape) == (24, 2, 16) and kv.planes["k"] is kv.k
    odd = pools.entry_cache(3)
    assert tuple(odd.k.shape) == (24, 2, 16) and tuple(odd.v.shape) == (24, 2, 8) and odd.block_size == 4


def test_a_fresh_state_is_what_the_spec_says():
    import torch

    from clockwork_amd.cache.pools import CachePools

    with pytest.raises(ValueError, match="fresh state"):
        StateSpec((4,), "float32", init=("ones",))
    filled, zeros = StateSpec((4,), "float32", init=("fill", 0.5)), StateSpec((4,), "float32")
    assert filled.group_key() != zeros.group_key()   # other beginnings, other pools
    groups = plan_groups([filled, zeros, filled])
    pools = CachePools(groups, 4, 2, 3, torch.float32, "cpu")
    # three slots for requests, the spare one, the template
    assert tuple(pools.state[0].shape) == (2, 5, 4) and tuple(pools.state[1].shape) == (1, 5, 4)
    assert bool((pools.state[0] == 0.5).all()) and bool((pools.state[1] == 0).all())
    pools.set_fresh_state(2, torch.arange(4.0))
    assert pools.state[0][1, 4].tolist() == [0.0, 1.0, 2.0, 3.0] and pools.state[0][0, 4].tolist() == [0.5] * 4
