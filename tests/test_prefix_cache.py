"""The prefix cache: the reference's radix-cache vectors (tests/test_radix.py) on our block trie."""

import random

import pytest

from clockwork_amd.cache import CacheManager, PrefixCache, plan_groups
from clockwork_amd.config.spec import KVPagesSpec

BS = 4


def setup(num_blocks=64, block_size=BS, enabled=True):
    m = CacheManager(plan_groups([KVPagesSpec(1, 16)]), block_size, num_blocks)
    return m, PrefixCache(block_size, m.share_handle, m.drop_handle, enabled=enabled)


def pages(m, n):
    return [(p,) for p in m.pools[0].take_many(n)]


def drop(m, handles):
    for h in handles:
        m.drop_handle(h)


def ref(m, handle):
    return m.pools[0].refcount(handle[0])


def test_match_on_an_empty_cache():
    _, cache = setup()
    r = cache.match(list(range(10)))
    assert (r.num_tokens, r.handles) == (0, [])
    assert (cache.stats.queries, cache.stats.prompt_tokens, cache.stats.hit_tokens) == (1, 10, 0)


def test_insert_keeps_whole_blocks_only():
    # tests/test_radix.py:44-56: 35 tokens, blocks of 16 -> 2 blocks stored, 32 tokens matched
    m, cache = setup(num_blocks=8, block_size=16)
    tokens = list(range(35))
    hs = pages(m, 3)
    assert cache.insert(tokens, hs) == 2
    assert cache.num_blocks() == 2
    assert [ref(m, h) for h in hs] == [2, 2, 1]
    r = cache.match(tokens)
    assert r.num_tokens == 32 and r.handles == hs[:2]


def test_a_match_never_covers_the_whole_sequence():
    # tests/test_radix.py:59-70
    m, cache = setup()
    tokens = list(range(8))
    hs = pages(m, 2)
    cache.insert(tokens, hs)
    r = cache.match(tokens)
    assert r.num_tokens == BS and r.handles == [hs[0]]
    r2 = cache.match(tokens + [99])
    assert r2.num_tokens == 8 and r2.handles == hs
    assert cache.match(tokens[:BS]).num_tokens == 0
    assert cache.match([]).num_tokens == 0


def test_a_match_takes_a_hold_per_block_and_release_can_give_them_back():
    m, cache = setup()
    hs = pages(m, 2)
    cache.insert(list(range(8)), hs)
    r = cache.match(list(range(8)) + [99])
    assert [ref(m, h) for h in r.handles] == [3, 3]
    cache.release(r, drop_holds=True)
    assert [ref(m, h) for h in hs] == [2, 2]


def test_branches_share_their_common_blocks():
    # tests/test_radix.py:85-107: the second branch keeps its own duplicates of the shared part
    m, cache = setup()
    a = [0] * 4 + [1] * 4 + [2] * 4
    b = [0] * 4 + [1] * 4 + [3] * 4
    ha, hb = pages(m, 3), pages(m, 3)
    assert cache.insert(a, ha) == 3
    assert cache.insert(b, hb) == 1
    assert cache.num_blocks() == 4
    assert [ref(m, h) for h in ha] == [2, 2, 2]
    assert [ref(m, h) for h in hb] == [1, 1, 2]
    r = cache.match(a + [9])
    assert (r.num_tokens, r.handles) == (12, ha)
    cache.release(r, drop_holds=True)
    r = cache.match(b + [9])
    assert (r.num_tokens, r.handles) == (12, [ha[0], ha[1], hb[2]])
    cache.release(r, drop_holds=True)


def test_divergence_inside_the_first_block():
    m, cache = setup()
    a = [1, 0, 0, 0, 7, 7, 7, 7]
    b = [1, 9, 9, 9, 8, 8, 8, 8]
    ha, hb = pages(m, 2), pages(m, 2)
    cache.insert(a, ha)
    cache.insert(b, hb)
    r = cache.match(a + [5])
    assert (r.num_tokens, r.handles) == (8, ha)
    r = cache.match(b + [5])
    assert (r.num_tokens, r.handles) == (8, hb)


def test_eviction_takes_the_oldest_unlocked_leaf_and_spares_locked_paths():
    m, cache = setup()
    old = pages(m, 2)
    new = pages(m, 2)
    cache.insert([1] * 8, old)
    cache.insert([2] * 8, new)
    drop(m, old + new)  # the requests are gone: the trie alone holds the pages
    assert cache.evictable_blocks() == 4
    held = cache.match([2] * 8 + [0])  # locks the newer branch (and refreshes it)
    assert cache.evictable_blocks() == 2
    assert cache.evict(1) == 1
    assert ref(m, old[1]) == 0 and ref(m, old[0]) == 1  # the leaf went first
    assert cache.evict(10) == 1  # the rest of the old branch; the locked one survives
    assert cache.num_blocks() == 2 and [ref(m, h) for h in new] == [2, 2]
    cache.release(held, drop_holds=True)
    assert cache.evict(10) == 2
    assert m.num_free_blocks() == 64


def test_lru_order():
    m, cache = setup()
    a, b, c = pages(m, 1), pages(m, 1), pages(m, 1)
    cache.insert([1] * 4, a)
    cache.insert([2] * 4, b)
    cache.insert([3] * 4, c)
    drop(m, a + b + c)
    cache.release(cache.match([1] * 4 + [0]), drop_holds=True)  # touch a
    assert cache.evict(1) == 1 and ref(m, b[0]) == 0
    assert cache.evict(1) == 1 and ref(m, c[0]) == 0
    assert ref(m, a[0]) == 1


def test_hit_rate_arithmetic_and_disabled_cache():
    # tests/test_llm_engine.py:185-193: four 19-token prompts that share 16 tokens
    m, cache = setup()
    prompts = [[5] * 16 + [i, i, i] for i in range(4)]
    for prompt in prompts:
        r = cache.match(prompt)
        hs = r.handles + pages(m, 5 - len(r.handles))
        cache.insert(prompt, hs[:4])
    assert (cache.stats.queries, cache.stats.prompt_tokens, cache.stats.hit_tokens) == (4, 76, 48)
    assert cache.stats.hit_rate == 48 / 76
    m2, off = setup(enabled=False)
    hs = pages(m2, 2)
    assert off.insert(list(range(8)), hs) == 0
    assert off.match(list(range(8)) + [1]).num_tokens == 0


def test_reset_drops_every_hold():
    m, cache = setup()
    hs = pages(m, 3)
    cache.insert(list(range(12)), hs)
    drop(m, hs)
    cache.reset()
    assert m.num_free_blocks() == 64 and cache.num_blocks() == 0


def test_fuzz_against_a_dict_of_prefixes_with_a_refcount_audit():
    # tests/test_radix.py:267-362 in spirit: reference model = {block-aligned prefix: handle}
    rng = random.Random(3)
    m, cache = setup(num_blocks=200)
    model: dict[tuple, tuple] = {}
    holds: list = []  # (match, extra handles owned by the "request")
    for _ in range(600):
        op = rng.random()
        tokens = [rng.randint(0, 2) for _ in range(rng.randint(1, 20))]
        if op < 0.45:
            r = cache.match(tokens)
            want = []
            limit = (len(tokens) - 1) // BS
            for b in range(limit):
                h = model.get(tuple(tokens[: (b + 1) * BS]))
                if h is None:
                    break
                want.append(h)
            assert r.handles == want and r.num_tokens == len(want) * BS
            n_full = len(tokens) // BS
            extra = n_full - len(r.handles)
            if extra > m.num_free_blocks():
                cache.release(r, drop_holds=True)
                continue
            own = pages(m, extra)
            cache.insert(tokens, r.handles + own)
            for b in range(n_full):
                model.setdefault(tuple(tokens[: (b + 1) * BS]), (r.handles + own)[b])
            holds.append((r, r.handles + own))
        elif op < 0.8 and holds:
            r, hs = holds.pop(rng.randrange(len(holds)))
            cache.release(r)
            drop(m, hs)
        else:
            before = cache.num_blocks()
            gone = cache.evict(rng.randint(1, 4))
            assert cache.num_blocks() == before - gone
            # rebuild the model from what the trie still matches
            model = {k: v for k, v in model.items() if _stored(cache, k)}
        # refcount = 1 for the trie + one per request holding the page
        counts: dict[tuple, int] = {}
        for h in model.values():
            counts[h] = counts.get(h, 0) + 1
        for _, hs in holds:
            for h in hs:
                counts[h] = counts.get(h, 0) + 1
        for page in range(200):
            assert m.pools[0].refcount(page) == counts.get((page,), 0)
    for r, hs in holds:
        cache.release(r)
        drop(m, hs)
    cache.reset()
    assert m.num_free_blocks() == 200


def _stored(cache, prefix) -> bool:
    node = cache._root
    for b in range(len(prefix) // BS):
        node = node.children.get(tuple(prefix[b * BS : (b + 1) * BS]))
        if node is None:
            return False
    return True
