"""The cache manager on the host: no page lost, held twice or freed twice."""
import random

import numpy as np
import pytest

from zse_amd.cache import CacheManager, GroupInfo, OutOfPages, OutOfSlots, PagePool, StateSlots, group_needs
from zse_amd.parts.base import PagedKV, StateNeed


def manager(pages=8, page=4, window=8, seqs=4, max_len=256, both=True):
    groups = [GroupInfo(window, [0], pages)] + ([GroupInfo(None, [1], pages)] if both else [])
    return CacheManager(groups, page, seqs, max_len, slot_bytes=16)


def test_pool_alloc_free_exhaustion_and_double_free():
    p = PagePool(3)
    a, b, c = p.alloc("x"), p.alloc("x"), p.alloc("y")
    assert sorted((a, b, c)) == [0, 1, 2] and p.free_pages == 0
    with pytest.raises(OutOfPages):
        p.alloc("z")
    p.free(b, "x")
    assert p.alloc("z") == b                     # the page freed last is used again first
    with pytest.raises(RuntimeError):
        p.free(a, "y")                           # not the owner
    p.free(a, "x")
    with pytest.raises(RuntimeError):
        p.free(a, "x")                           # freed twice
    p.check()


def test_groups_come_from_needs():
    needs = [PagedKV(2, 16, 8), PagedKV(2, 16, None), None, PagedKV(2, 16, 8), StateNeed(32)]
    g = group_needs(needs)
    assert [(x.window, x.calls) for x in g] == [(8, [0, 3]), (None, [1])]


def test_pages_follow_length_as_in_the_reference_vector():
    # ceil(20/4) = 5 pages, 6 after one more token (reference tests/test_kv_cache.py:326-358)
    m = manager(pages=16, window=1000)
    m.add("r")
    assert m.reserve("r", 20)
    assert [len(m.table("r", g)) for g in (0, 1)] == [5, 5]
    m.commit("r", 20)
    assert m.reserve("r", 21)
    assert [len(m.table("r", g)) for g in (0, 1)] == [6, 6]
    m.check()


def test_reserve_is_all_or_nothing():
    m = manager(pages=4)
    m.add("a"), m.add("b")
    assert m.reserve("a", 12)                    # 3 pages in each group
    before = [p.free_pages for p in m.pools]
    assert not m.reserve("b", 8)                 # needs 2, one is free
    assert [p.free_pages for p in m.pools] == before
    assert m.table("b", 0) == [] and m.table("b", 1) == []
    assert m.pages_short("b", 8) == [1, 1]
    m.check()


def test_window_release_rule():
    # page j goes back iff (j+1)*page - 1 <= n - window
    m = manager(pages=16, page=4, window=8)
    m.add("r")
    m.reserve("r", 23)
    freed = m.commit("r", 23)
    # n - W = 15: pages 0..3 hold positions up to 15 -> released; page 4 (16..19) stays
    assert len(freed[0]) == 4 and freed[1] == []
    t = m.table("r", 0)
    assert t[:4] == [-1] * 4 and all(p >= 0 for p in t[4:])
    assert all(p >= 0 for p in m.table("r", 1))          # the all-keys group keeps everything
    # every key a later query can see is still there: query at n sees n-W+1 .. n
    assert (23 - 8 + 1) // 4 >= 4
    assert m.computed("r") == 23                          # a release never shortens the request
    with pytest.raises(RuntimeError):
        m.slot_mapping("r", 0, 12, 4)                     # a released page cannot be written
    sm = m.slot_mapping("r", 0, 21, 2)
    assert list(sm) == [t[5] * 4 + 1, t[5] * 4 + 2]
    assert m.slot_of("r", 0, 22) == sm[1] and m.slot_of("r", 1, 3) == m.table("r", 1)[0] * 4 + 3
    with pytest.raises(RuntimeError):
        m.slot_of("r", 0, 15)                             # one position on a released page
    m.check()


def test_release_returns_everything_and_twice_is_a_no_op():
    m = manager()
    s = m.add("r")
    m.reserve("r", 9)
    m.release("r")
    m.release("r")
    assert all(p.free_pages == p.num_pages for p in m.pools) and m.slots.free_slots == 4
    assert m.add("q") == s                                # the slot is used again
    m.check()


def test_slots_run_out_and_limits_hold():
    m = manager(seqs=2)
    m.add(1), m.add(2)
    with pytest.raises(OutOfSlots):
        m.add(3)
    with pytest.raises(ValueError):
        m.add(1)
    with pytest.raises(ValueError):
        m.reserve(1, 257)                                 # beyond the longest context
    s = StateSlots(2, 8)
    s.acquire("a")
    with pytest.raises(ValueError):
        s.acquire("a")


def test_table_row_is_padded_with_holes():
    m = manager(pages=8, page=4, window=4)
    m.add("r")
    m.reserve("r", 10)
    m.commit("r", 10)
    row = np.full(m.max_blocks, 7, dtype=np.int32)
    m.fill_table_row("r", 0, row)
    assert row[0] == -1 and row[1] >= 0 and row[2] >= 0 and (row[3:] == -1).all()


@pytest.mark.parametrize("seed", range(6))
def test_random_orders_keep_every_invariant(seed):
    rng = random.Random(seed)
    page, window = rng.choice([(4, 8), (8, 16), (4, 5), (16, 4)])
    m = manager(pages=rng.randint(6, 24), page=page, window=window, seqs=4, max_len=400)
    live, next_id = {}, 0
    visible_ok = 0
    for _ in range(600):
        op = rng.random()
        if op < 0.25 and len(live) < 4:
            m.add(next_id)
            live[next_id] = 0
            next_id += 1
        elif op < 0.85 and live:
            r = rng.choice(list(live))
            n = rng.choice([1, 1, 1, 2, 3, 7, 13, 30])
            if live[r] + n > 400:
                continue
            if m.reserve(r, live[r] + n):
                # every position the step's tokens can see is on a held page
                lo = max(0, live[r] - window + 1)
                t0 = m.table(r, 0)
                assert all(t0[j] >= 0 for j in range(lo // page, -(-(live[r] + n) // page)))
                t1 = m.table(r, 1)
                assert all(p >= 0 for p in t1) and len(t1) == -(-(live[r] + n) // page)
                m.slot_mapping(r, 0, live[r], n), m.slot_mapping(r, 1, live[r], n)
                live[r] += n
                m.commit(r, live[r])
                visible_ok += 1
        elif live:
            r = rng.choice(list(live))
            m.release(r)
            del live[r]
        m.check()
        # windowed group never holds more than the window needs
        for r, n in live.items():
            held = sum(1 for p in m.table(r, 0) if p >= 0)
            assert held <= -(-window // page) + 1 + 30 // page + 1
    assert visible_ok > 50
    for r in list(live):
        m.release(r)
    m.check()
    assert all(p.free_pages == p.num_pages for p in m.pools) and m.slots.free_slots == 4


def test_attention_workspace_follows_the_models_limits():
    """The split attention's workspace is what its kernel asks for at the runner's limits:
    requests x heads x chunks of 64 keys x (head_dim + 2) floats.  At 64 requests of 8192
    tokens the two larger models need more than the 128 MB a fixed buffer once gave them."""
    from zse_amd.config import AttentionSpec, RotarySpec
    from zse_amd.parts import build_part
    from zse_amd.runtime import build
    from zse_amd.runtime.device import KernelLibrary
    try:
        k = KernelLibrary(build.ensure("kernels_bf16", verbose=False), "bfloat16")
    except build.BuildError as e:
        pytest.skip(f"the kernel library cannot be built here: {e}")
    for nh, nkv, hd, want in [(8, 4, 256, 67633152), (16, 8, 256, 135266304), (32, 16, 128, 136314880)]:
        spec = AttentionSpec(1024, nh, nkv, hd, hd ** -0.5, 50.0, None, RotarySpec(hd, hd, 1e4),
                             {r: r for r in "qkvo"})
        part = build_part("mixer", spec)
        need = part.prepare(k, "bfloat16", 64, 8192, 16)
        assert need == want == 64 * nh * 128 * (hd + 2) * 4
        assert part.decode_chunk == 64
        assert part.prepare(k, "bfloat16", 1, 4096, 16) == nh * 64 * (hd + 2) * 4
        assert part.decode_chunk == (32 if nkv * 64 <= 512 else 64)      # one request: finer cuts while waves are few
        assert part.prepare(k, "float32", 64, 8192, 16) == 0           # the plain kernel needs none
    # a context the decode kernel cannot join is refused when the runner is made, with the numbers
    with pytest.raises(ValueError, match="longest context"):
        part.prepare(k, "bfloat16", 64, 300000, 16)


def test_a_pool_whose_ids_begin_at_one_and_the_page_a_step_begins_to_fill():
    from zse_amd.cache.manager import CacheManager, GroupInfo
    from zse_amd.cache.pages import PagePool
    pool = PagePool(3, first_id=1)
    got = [pool.alloc("a") for _ in range(3)]
    assert got == [1, 2, 3] and pool.free_pages == 0
    with pytest.raises(ValueError):
        pool.free(0, "a")
    pool.free(2, "a")
    pool.check()
    assert pool.alloc("b") == 2

    m = CacheManager([GroupInfo(8, [0], 6), GroupInfo(None, [1], 6)], page_size=4, max_seqs=2, max_model_len=24,
                     first_page=1)
    m.add("r")
    assert m.reserve("r", 6)
    # 6 tokens: page 0 of the request is filled, its page 1 is begun and was never written
    assert m.untouched_page("r", 0, 6) == m.table("r", 0)[1] and m.untouched_page("r", 1, 6) == m.table("r", 1)[1]
    assert min(m.table("r", 0)) >= 1
    m.commit("r", 6)
    assert m.reserve("r", 7)
    assert m.untouched_page("r", 0, 7) is None          # the request wrote to that page in the step before
    m.commit("r", 7)
    assert m.reserve("r", 8) and m.untouched_page("r", 0, 8) is None      # a step that fills its last page
    m.commit("r", 8)
    assert m.reserve("r", 9)
    assert m.untouched_page("r", 0, 9) == m.table("r", 0)[2]
    m.commit("r", 9)
    # a step of many tokens: only the page it ends in can be left half filled
    assert m.reserve("r", 22) and m.untouched_page("r", 1, 22) == m.table("r", 1)[5]
    m.check()
