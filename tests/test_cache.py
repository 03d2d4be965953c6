"""The cache manager on the host: allocator, block tables, groups, window pages,
state slots; no page lost, held twice or freed twice under random orders of requests."""
import random

import pytest

from infernum_amd.cache import (NO_PAGE, CacheConfig, CacheManager, PageAllocator, PageError,
                                StateSlotPool, pages_for)
from infernum_amd.parts import CacheSpec, StateSpec

FULL = CacheSpec("full", 2, 16)
WIN = CacheSpec("window", 2, 16, window=10)


def manager(needs, page_size=4, num_pages=16, slots=4, cache_of=None):
    return CacheManager(needs, cache_of or [None] * len(needs),
                        CacheConfig(page_size=page_size, num_pages=num_pages, num_state_slots=slots), device=None)


# ---- allocator (infernum/src/block_allocator.rs:204-429) ---------------------------------
def test_allocator_hands_out_every_page_once_then_nothing():
    a = PageAllocator(4)
    got = [a.allocate() for _ in range(4)]
    assert sorted(got) == [0, 1, 2, 3] and a.allocate() is None and a.num_free == 0
    assert a.allocate_many(1) is None


def test_allocator_reuses_the_page_freed_last():
    a = PageAllocator(8)
    p = [a.allocate() for _ in range(3)]
    a.free(p[1])
    assert a.allocate() == p[1]
    a.free(p[0]); a.free(p[2])
    assert a.allocate() == p[2] and a.allocate() == p[0]


def test_allocator_refuses_double_free_and_pages_outside_the_pool():
    a = PageAllocator(4)
    p = a.allocate()
    a.free(p)
    with pytest.raises(PageError, match="twice"):
        a.free(p)
    with pytest.raises(PageError, match="outside"):
        a.free(4)
    with pytest.raises(PageError, match="outside"):
        a.free(-1)
    with pytest.raises(PageError, match="twice"):
        a.free(3)                      # never handed out
    with pytest.raises(ValueError):
        PageAllocator(0)


def test_allocate_many_is_all_or_nothing():
    a = PageAllocator(5)
    assert a.allocate_many(6) is None and a.num_free == 5
    assert len(a.allocate_many(5)) == 5 and a.num_free == 0


def test_pages_for_table():
    # block_allocator.rs: 0,1,16,17,32,33 tokens -> 0,1,1,2,2,3 blocks of 16
    assert [pages_for(n, 16) for n in (0, 1, 16, 17, 32, 33)] == [0, 1, 1, 2, 2, 3]


# ---- requests ---------------------------------------------------------------------------
def test_block_table_lifecycle():
    m = manager([(FULL, None)], page_size=4, num_pages=8)
    assert m.admit("a")
    assert m.num_tokens("a") == 0 and m.block_table(0, "a").pages == []
    assert m.pages_needed("a", 5) == [2] and m.pages_needed("never seen", 9) == [3]
    assert m.reserve("a", 5)
    assert len(m.block_table(0, "a").pages) == 2 and m.free_pages() == 6
    assert m.token_slots(0, "a", 0, 5).tolist() == [p * 4 + o for p, o in
                                                    zip([m.block_table(0, "a").pages[0]] * 4 + [m.block_table(0, "a").pages[1]], [0, 1, 2, 3, 0])]
    m.commit("a", 5)
    assert m.num_tokens("a") == 5
    assert m.pages_needed("a", 3) == [0] and m.pages_needed("a", 4) == [1]     # 3 more fit the second page
    assert m.reserve("a", 3) and m.free_pages() == 6
    m.commit("a", 3)
    m.check()
    m.release("a")
    assert m.free_pages() == 8 and not m.has("a")
    m.check()


def test_reserve_is_all_or_nothing_and_storing_without_pages_fails():
    m = manager([(FULL, None)], page_size=4, num_pages=3)
    m.admit("a"); m.admit("b")
    assert m.reserve("a", 8)
    assert not m.reserve("b", 8) and m.block_table(0, "b").pages == [] and m.free_pages() == 1
    assert m.tokens_that_fit("b") == 4 and m.tokens_that_fit("a") == 12 and m.tokens_that_fit(None, [1]) == 0
    with pytest.raises(PageError):
        m.commit("b", 1)
    with pytest.raises(PageError):
        m.token_slots(0, "b", 0, 1)


def test_requests_twice_and_unknown():
    m = manager([(FULL, None)])
    m.admit("a")
    with pytest.raises(PageError, match="twice"):
        m.admit("a")
    with pytest.raises(PageError, match="not admitted"):
        m.release("zzz")
    m.release("a")
    with pytest.raises(PageError):
        m.release("a")


def test_state_slots():
    p = StateSlotPool(2)
    a, b = p.acquire(), p.acquire()
    assert {a, b} == {0, 1} and p.acquire() is None
    p.release(a)
    with pytest.raises(PageError):
        p.release(a)
    with pytest.raises(PageError):
        p.release(5)
    assert p.acquire() == a
    m = manager([(FULL, StateSpec((3,)))], slots=2)
    assert m.admit("a") and m.admit("b") and not m.admit("c")
    assert m.state_slot("a") != m.state_slot("b")
    m.release("a")
    assert m.admit("c")
    m.check()


# ---- groups --------------------------------------------------------------------------------
def test_layers_with_equal_needs_share_a_group_and_a_reader_owns_nothing():
    needs = [(FULL, None), (WIN, None), (FULL, None), (None, None)]
    m = manager(needs, cache_of=[None, None, None, 0])
    assert len(m.groups) == 2
    assert m.groups[0].entries == [0, 2] and m.groups[1].entries == [1]
    v = m.views()
    assert (v[0].group, v[1].group, v[2].group, v[3].group) == (0, 1, 0, 0)
    assert v[3].writable is False and v[0].writable is True


def test_window_group_gives_pages_back_as_the_window_passes_them():
    m = manager([(FULL, None), (WIN, None)], page_size=4, num_pages=8)
    m.admit("a")
    for step in range(30):
        assert m.reserve("a", 1), step
        m.commit("a", 1)
        m.check()
        n = m.num_tokens("a")
        t = m.block_table(1, "a")
        # the next query stands at position n and sees keys n-9 .. n: pages below (n-9)//4 are gone
        first_needed = max(0, n - 10 + 1) // 4
        assert t.first_live == min(first_needed, len(t.pages))
        assert all(p == NO_PAGE for p in t.pages[:t.first_live])
        assert all(p != NO_PAGE for p in t.pages[t.first_live:])
        assert len(t.live_pages()) <= 4                      # a window of 10 never needs more than 4 pages of 4
    assert len(m.block_table(0, "a").live_pages()) == 8          # the full group keeps everything
    assert not m.reserve("a", 3)                                 # and is what runs out first
    m.release("a")
    assert m.free_pages(0) == 8 and m.free_pages(1) == 8


def test_window_pages_of_a_long_portion_are_kept_until_stored():
    m = manager([(WIN, None)], page_size=4, num_pages=8)
    m.admit("a")
    assert m.reserve("a", 30)                # one portion of 30 tokens needs all its 8 pages at once
    assert m.free_pages() == 0
    m.commit("a", 30)
    assert m.free_pages() == 5               # keys 21..29 and the next token: pages 5, 6, 7
    m.check()


# ---- random orders ---------------------------------------------------------------------------
@pytest.mark.parametrize("seed", range(6))
def test_random_orders_lose_no_page(seed):
    rng = random.Random(seed)
    needs = [(FULL, None), (WIN, None), (FULL, StateSpec((2,)))]
    m = manager(needs, page_size=rng.choice((2, 4, 8)), num_pages=rng.choice((6, 16, 40)), slots=5)
    live, next_id = {}, 0
    for it in range(600):
        op = rng.random()
        if op < 0.2 and len(live) < 5:
            assert m.admit(next_id)
            live[next_id] = 0
            next_id += 1
        elif op < 0.85 and live:
            r = rng.choice(list(live))
            n = rng.choice((1, 1, 1, 2, 3, 7, 20))
            before = [g.allocator.num_free for g in m.groups]
            need = m.pages_needed(r, n)
            ok = m.reserve(r, n)
            assert ok == all(a <= b for a, b in zip(need, before))
            if ok:
                assert [b - g.allocator.num_free for b, g in zip(before, m.groups)] == need
                m.commit(r, n)
                live[r] += n
                assert m.num_tokens(r) == live[r]
            else:
                assert [g.allocator.num_free for g in m.groups] == before      # nothing was taken
        elif live:
            r = rng.choice(list(live))
            m.release(r)
            del live[r]
        m.check()
        assert sorted(m.requests()) == sorted(live)
    for r in list(live):
        m.release(r)
    m.check()
    assert all(g.allocator.num_free == g.allocator.num_pages for g in m.groups)
    assert m.slots.num_free == 5


def test_a_step_that_fails_leaves_the_cache_as_it_was():
    """Engine.step: when the forward pass raises (here: no GPU, so the first kernel call does), requests that
    came with the step are gone again and the others hold what they held before."""
    import torch
    import tiny_models as TM
    from infernum_amd import CacheConfig, Engine
    from infernum_amd.kernels.api import KernelError
    from infernum_amd.weights.random_init import _cpu_model
    if torch.cuda.is_available():
        pytest.skip("the forward pass must fail for this test: it needs a machine without a GPU")
    model = _cpu_model(TM.tiny_config("C"), torch.float32)       # two groups: all keys, and a window
    eng = Engine(model, CacheConfig(page_size=4, num_pages=16, num_state_slots=3))
    cache = eng.cache
    cache.admit("old")
    assert cache.reserve("old", 6)
    cache.commit("old", 6)
    free_before = [cache.free_pages(g) for g in range(len(cache.groups))]
    table_before = [cache.block_table(g, "old").pages for g in range(len(cache.groups))]
    for entries in ([("new", [1, 2, 3, 4, 5], [4])],                       # a request that comes with the step
                    [("old", [7], [0])],                                   # one that was there, a single token
                    [("old", [7, 8, 9, 1, 2, 3, 4], [6]), ("new", [5, 6], [])]):   # both, more pages for "old"
        with pytest.raises(KernelError):
            eng.step(entries)
        assert cache.requests() == ["old"] and cache.num_tokens("old") == 6
        assert [cache.free_pages(g) for g in range(len(cache.groups))] == free_before
        assert [cache.block_table(g, "old").pages for g in range(len(cache.groups))] == table_before
        assert cache.slots.num_free == 2
        cache.check()
    assert eng.steps_run == 0


def test_pools_are_what_the_mixers_declare():
    """A page's payload comes from the mixer's CacheSpec: named tensors with a per-token shape and the axis
    that the page's tokens run along; keys and values in the attention kernels' layouts are the default."""
    import torch
    from infernum_amd.parts import CacheSpec, PageTensor
    latent = CacheSpec("window", window=6, payload=(PageTensor("latent", (12,), 0, torch.float32),
                                                    PageTensor("scale", (), 0)))
    kv = CacheSpec("full", 2, 16)
    assert [(t.name, t.shape, t.token_axis) for t in kv.payload] == [("k", (2, 16), 1), ("v", (2, 16), 2)]
    m = CacheManager([(latent, None), (kv, None), (None, None)], [None, None, 1],
                     CacheConfig(page_size=4, num_pages=8, poison_freed_pages=True), dtype=torch.bfloat16,
                     device=torch.device("cpu"))
    shapes = [{k: (tuple(v.shape), v.dtype) for k, v in p.items()} for p in m.pages]
    assert shapes == [{"latent": ((8, 4, 12), torch.float32), "scale": ((8, 4), torch.bfloat16)},
                      {"k": ((8, 2, 4, 16), torch.bfloat16), "v": ((8, 2, 16, 4), torch.bfloat16)}, {}]
    views = m.views()
    assert views[0].k_pages is None and views[0].pages["latent"] is m.pages[0]["latent"]
    assert views[2].pages is views[1].pages and not views[2].writable and views[2].k_pages is m.pages[1]["k"]
    # freed pages are poisoned in every pool of their group
    m.admit("a")
    assert m.reserve("a", 9)
    m.commit("a", 9)
    pages = {g: m.block_table(g, "a").pages for g in range(2)}
    m.release("a")
    assert all(bool(m.pages[0]["latent"][p].isnan().all()) and bool(m.pages[0]["scale"][p].isnan().all())
               for p in pages[0] if p >= 0)
    assert all(bool(m.pages[1]["k"][p].isnan().all()) for p in pages[1])
    with pytest.raises(ValueError):
        CacheSpec("full")
    with pytest.raises(ValueError):
        CacheSpec("full", payload=(PageTensor("x", (3,)), PageTensor("x", (4,))))
    with pytest.raises(ValueError):
        PageTensor("x", (3,), token_axis=2).pool_shape(4, 4)
