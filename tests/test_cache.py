"""The cache manager on the CPU: no page lost, held twice or freed twice, under
random orders of requests; block tables; windows; slots."""

import random

import pytest

from zig_ai_amd.cache import FREED, CacheManager, OutOfPages, OutOfSlots, Pool, PoolError
from zig_ai_amd.parts import PagedNeed, StateNeed


def manager(num_pages=16, page_size=4, num_slots=4, window=0, extra=None):
    needs = {0: StateNeed((8, 3)), 1: PagedNeed.kv(2, 16, 0), 2: StateNeed((8, 3)), 3: PagedNeed.kv(2, 16, 0)}
    if window:
        needs[4] = PagedNeed.kv(2, 16, window)
    needs.update(extra or {})
    return CacheManager(needs, page_size, num_pages, num_slots, allocate=False)


def test_pool_counts_like_the_reference():
    """/root/reference/tests/test_paged_attention.zig:18-30: 16 -> alloc -> 15 -> release -> 16."""
    p = Pool(16)
    assert p.free_count == 16
    page = p.take("x")
    assert p.free_count == 15 and p.owner_of(page) == "x"
    p.give(page, "x")
    assert p.free_count == 16
    p.check()


def test_pool_refuses_double_free_and_foreign_free():
    p = Pool(4)
    a = p.take("x")
    with pytest.raises(PoolError, match="belongs"):
        p.give(a, "y")
    p.give(a, "x")
    with pytest.raises(PoolError, match="twice"):
        p.give(a, "x")
    with pytest.raises(PoolError, match="exist"):
        p.give(9, "x")
    for _ in range(4):
        p.take("z")
    with pytest.raises(OutOfPages):
        p.take("z")
    with pytest.raises(OutOfPages):
        Pool(2).take_many("q", 3)


def test_block_table_growth_like_the_reference():
    """/root/reference/tests/test_paged_attention.zig:32-58 and
    test_paged_attention_gpu.zig:51,294: 5 tokens at page 4 -> 2 pages, 7 -> 2, 9 -> 3;
    40 at 16 -> 3; 4096 at 16 -> 256."""
    for tokens, page, want in [(5, 4, 2), (7, 4, 2), (9, 4, 3), (40, 16, 3), (4096, 16, 256)]:
        m = CacheManager({0: PagedNeed.kv(1, 16)}, page, 300, 1, allocate=False)
        m.admit("r")
        m.reserve("r", tokens)
        assert len(m.table("r", 0)) == want
    m = manager(page_size=4)
    m.admit("r")
    m.reserve("r", 4)
    m.commit("r", 4)
    assert len(m.table("r", 0)) == 1
    m.reserve("r", 1)                      # the fifth token opens a new page
    assert len(m.table("r", 0)) == 2
    m.commit("r", 1)
    assert m.token_slots("r", 0, 0, 5) == [m.table("r", 0)[0] * 4 + i for i in range(4)] + \
        [m.table("r", 0)[1] * 4]


def test_groups_and_views():
    m = manager(window=6)
    assert len(m.groups) == 2                      # all keys; a window of keys
    assert m.groups[0].cache_ids == [1, 3] and m.groups[1].cache_ids == [4]
    assert m.view(1).kind == "paged" and m.view(1).group == 0 and m.view(4).group == 1
    assert m.view(0).kind == "state" and m.view(7).kind == "none"
    assert m.bytes_per_slot == 2 * 8 * 3 * 4


def test_planes_and_typed_state_in_memory():
    """What mixers declare decides the memory: planes of different sizes in one page, a
    storage type per need, state of any type; on the CPU here, the layout is the same."""
    import torch
    latent = PagedNeed(((1, 24),), dtype=torch.float32)              # one vector per token
    uneven = PagedNeed(((2, 16), (2, 8), (1, 4)))                    # three planes, different sizes
    needs = {"kv": PagedNeed.kv(2, 16), ("a", "mixer"): latent, ("b", "mixer"): latent, "u": uneven,
             "count": StateNeed((1,), dtype=torch.int32), "conv": StateNeed((8, 3)),
             "flag": StateNeed((5,), dtype=torch.uint8)}
    m = CacheManager(needs, 4, {PagedNeed.kv(2, 16): 6, latent: 5, uneven: 3}, 3,
                     device=torch.device("cpu"), dtype=torch.bfloat16)
    assert [len(g.cache_ids) for g in m.groups] == [1, 2, 1]
    kv, lat, une = m.groups
    assert kv.memory.shape == (1, 6, 4 * 2 * 2 * 16) and kv.memory.dtype == torch.bfloat16
    assert lat.memory.shape == (2, 5, 4 * 24) and lat.memory.dtype == torch.float32
    assert une.memory.shape == (1, 3, 4 * (32 + 16 + 4))
    assert kv.kv.shape == (1, 6, 2, 2, 4, 16) and lat.kv is None and une.kv is None
    v = m.view("kv")
    assert v.kv.shape == (6, 2, 2, 4, 16) and [tuple(p.shape) for p in v.planes] == [(6, 2, 4, 16)] * 2
    v.planes[1][3, 1, 2, 5] = 7.0                  # the second plane IS the values' half of kv
    assert float(v.kv[3, 1, 1, 2, 5]) == 7.0
    second = m.view(("b", "mixer"))
    assert second.kv is None and tuple(second.planes[0].shape) == (5, 1, 4, 24)
    second.planes[0][2, 0, 1, 3] = 1.5
    assert float(lat.memory[1, 2, 1 * 24 + 3]) == 1.5 and float(lat.memory[0].abs().sum()) == 0.0
    shapes = [tuple(p.shape) for p in m.view("u").planes]
    assert shapes == [(3, 2, 4, 16), (3, 2, 4, 8), (3, 1, 4, 4)]
    m.view("u").planes[2][1, 0, 3, 2] = 2.0         # the last element but one row of page 1
    assert float(une.memory[0, 1, 4 * 48 + 3 * 4 + 2]) == 2.0
    # a page more in every group costs the bytes of one page of every entry
    assert CacheManager.bytes_per_page_index(needs, 4, torch.bfloat16) == \
        4 * (64 * 2 + 24 * 4 * 2 + 52 * 2)
    # state: typed windows of one row of bytes per slot, each 16-byte aligned
    count, conv, flag = m.view("count").state, m.view("conv").state, m.view("flag").state
    assert (count.dtype, conv.dtype, flag.dtype) == (torch.int32, torch.float32, torch.uint8)
    assert tuple(count.shape) == (3, 1) and tuple(conv.shape) == (3, 8, 3) and tuple(flag.shape) == (3, 5)
    assert m.bytes_per_slot == 16 + 96 + 16
    slot = m.admit("r")
    count[slot, 0] = 41
    conv[slot] = 2.5
    flag[slot] = 9
    m.release("r")
    assert m.admit("again") == slot                 # the slot comes back cleared
    assert int(count[slot, 0]) == 0 and float(conv[slot].abs().sum()) == 0.0 and int(flag[slot].sum()) == 0
    with pytest.raises(ValueError):
        CacheManager({0: PagedNeed(())}, 4, 4, 1, allocate=False)


def test_state_that_starts_elsewhere_than_zero():
    """A state need may name its starting value: a running maximum at -inf, a product at 1,
    a counter at -1; every new request finds it, also in a slot another request used, and
    the entries beside it still start at zero."""
    import math

    import torch
    needs = {"top": StateNeed((4,), init=-math.inf), "conv": StateNeed((2, 3)),
             "scale": StateNeed((2,), dtype=torch.float32, init=1.0),
             "last": StateNeed((1,), dtype=torch.int32, init=-1)}
    m = CacheManager(needs, 4, 4, 2, device=torch.device("cpu"), dtype=torch.float32)
    top, conv, scale, last = (m.view(k).state for k in ("top", "conv", "scale", "last"))
    for name in ("a", "b"):
        slot = m.admit(name)
        assert bool(torch.isinf(top[slot]).all()) and float(top[slot].max()) < 0
        assert float(conv[slot].abs().sum()) == 0.0
        assert scale[slot].tolist() == [1.0, 1.0] and int(last[slot, 0]) == -1
        top[slot] = 3.0
        conv[slot] = 7.0
        scale[slot] = 0.5
        last[slot, 0] = 12
    m.release("a")
    slot = m.admit("c")                              # a's slot again
    assert bool(torch.isinf(top[slot]).all()) and float(conv[slot].abs().sum()) == 0.0
    assert scale[slot].tolist() == [1.0, 1.0] and int(last[slot, 0]) == -1
    other = m.slot_of("b")
    assert float(top[other, 0]) == 3.0 and int(last[other, 0]) == 12     # b's state is untouched


def test_reserve_is_all_or_nothing():
    m = manager(num_pages=4, window=6)
    m.admit("a")
    m.admit("b")
    m.reserve("a", 12)                              # 3 of 4 pages in both groups
    with pytest.raises(OutOfPages):
        m.reserve("b", 8)                           # needs 2
    assert m.table("b", 0) == [] and m.table("b", 1) == []
    assert not m.can_reserve("b", 8) and m.can_reserve("b", 4)
    assert not m.can_reserve("b", 4, spare={0: 1})
    m.check()


def test_window_gives_pages_back():
    m = manager(num_pages=8, page_size=4, window=6)
    m.admit("r")
    for step in range(40):
        m.reserve("r", 1)
        m.commit("r", 1)
        m.check()
        n = step + 1
        table = m.table("r", 1)
        first_needed = max(0, n - 6 + 1)
        for p, page in enumerate(table):
            assert (page == FREED) == ((p + 1) * 4 <= first_needed), (n, p)
        assert len(m.table("r", 0)) == (n + 3) // 4 and FREED not in m.table("r", 0)
        if n >= 32:
            break
    assert m.groups[1].pool.high_water <= 3           # never more than window/page + 2 pages
    with pytest.raises(PoolError, match="given back"):
        m.token_slots("r", 1, 0, 1)
    m.release("r")
    assert all(g.pool.free_count == g.pool.size for g in m.groups)


def test_commit_beyond_reservation_is_an_error():
    m = manager()
    m.admit("r")
    m.reserve("r", 3)
    with pytest.raises(PoolError, match="beyond"):
        m.commit("r", 5)


def test_slots():
    m = manager(num_slots=2)
    assert m.admit("a") != m.admit("b")
    with pytest.raises(OutOfSlots):
        m.admit("c")
    with pytest.raises(PoolError, match="already"):
        m.admit("a")
    m.release("a")
    m.admit("c")
    m.check()


@pytest.mark.parametrize("seed", range(8))
def test_random_orders_keep_the_books(seed):
    """Admissions, portions, decoding, finishing in random order: after every
    action free + owned = total, no page in two tables, tables match the pools."""
    rng = random.Random(seed)
    m = manager(num_pages=24, page_size=4, num_slots=5, window=rng.choice([0, 5, 9]))
    live, next_id = {}, 0
    for _ in range(600):
        action = rng.random()
        if action < 0.25 and len(live) < 5:
            m.admit(next_id)
            live[next_id] = 0
            next_id += 1
        elif action < 0.85 and live:
            r = rng.choice(list(live))
            n = rng.choice([1, 1, 1, 2, 3, 7, 16])
            try:
                m.reserve(r, n)
            except OutOfPages:
                victim = rng.choice(list(live))       # what a scheduler would do: evict one
                m.release(victim)
                del live[victim]
                m.check()
                continue
            m.commit(r, n)
            live[r] += n
            assert m.num_tokens(r) == live[r]
        elif live:
            r = rng.choice(list(live))
            m.release(r)
            del live[r]
        m.check()
        for g in m.groups:
            held = sum(1 for r in live for p in m.table(r, g.index) if p != FREED)
            assert held + g.pool.free_count == g.pool.size
    for r in list(live):
        m.release(r)
    m.check()
    assert all(g.pool.free_count == g.pool.size for g in m.groups)
    assert m.slots.free_count == 5
    assert m.pages_reused > 0


def test_scattered_pools_hand_out_every_page_once():
    """A cache made with scatter_pages hands its pages out in a fixed shuffled order:
    every page exactly once, the same order in every cache of that size, and the
    books stay right when pages come back."""
    orders = []
    for _ in range(2):
        m = CacheManager({0: PagedNeed.kv(1, 16)}, 4, 257, 2, allocate=False, scatter_pages=True)
        m.admit("r")
        m.reserve("r", 257 * 4)
        order = m.table("r", 0)
        assert sorted(order) == list(range(257))
        m.admit("s")
        with pytest.raises(OutOfPages):
            m.reserve("s", 1)
        m.release("r")
        m.check()
        assert m.groups[0].pool.free_count == 257
        orders.append(order)
    assert orders[0] == orders[1]
    assert orders[0] != list(range(257))
    runs = sum(1 for a, b in zip(orders[0], orders[0][1:]) if b == a + 1)
    assert runs < 16                                   # no long stretches in address order
    plain = CacheManager({0: PagedNeed.kv(1, 16)}, 4, 257, 2, allocate=False)
    plain.admit("r")
    plain.reserve("r", 40)
    assert plain.table("r", 0) == list(range(10))      # the default: 0, 1, 2 ...
