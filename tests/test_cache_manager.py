"""The host side of the cache: pages, block tables, slots (CPU only)."""

import random

import numpy as np
import pytest

from rapid_llm_amd.cache import NULL_PAGE, CacheError, CacheManager, GroupSpec, PagePool
from rapid_llm_amd.cache.storage import plan_groups
from rapid_llm_amd.parts.base import CacheNeed


def test_null_page_is_never_handed_out():
    pool = PagePool(5)  # rapid_llm/engine/block_pool.py:19-22
    pages = pool.take(4)
    assert sorted(pages) == [1, 2, 3, 4] and NULL_PAGE not in pages
    assert pool.take(1) is None and pool.num_free == 0


def test_short_pool_takes_nothing():
    pool = PagePool(4)
    assert pool.take(5) is None  # all or nothing (block_pool.py:234)
    assert pool.num_free == 3
    assert pool.take(0) == []


def test_double_free_and_foreign_pages_raise():
    pool = PagePool(4)
    (a,) = pool.take(1)
    pool.give_back([a])
    with pytest.raises(CacheError, match="twice"):
        pool.give_back([a])
    with pytest.raises(CacheError, match="null page"):
        pool.give_back([NULL_PAGE])
    with pytest.raises(CacheError, match="not in this pool"):
        pool.give_back([9])


def test_pages_given_back_are_taken_again_first():
    pool = PagePool(10)
    first = pool.take(3)
    pool.give_back(first)
    assert set(pool.take(3)) == set(first)


def _manager(num_pages=9, page=4, seqs=3, max_len=64, windows=(0,)):
    groups = [GroupSpec(i, w, (i,)) for i, w in enumerate(windows)]
    return CacheManager(groups, num_pages, page, seqs, max_len)


def test_reserve_maps_pages_and_is_all_or_nothing():
    m = _manager(num_pages=5)  # 4 usable pages of 4 positions
    assert m.admit("a") == 0
    assert m.reserve("a", 9)  # 3 pages
    assert len(m.pages_of("a", 0)) == 3 and m.reserved("a") == 9
    assert m.reserve("a", 12) and len(m.pages_of("a", 0)) == 3  # same page
    m.admit("b")
    before = (m.num_free_pages(), m.tables[0].copy())
    assert not m.reserve("b", 8)  # needs 2, 1 free: nothing changes
    assert m.num_free_pages() == before[0] and np.array_equal(m.tables[0], before[1])
    assert m.reserve("b", 4)
    m.check_invariants()
    m.release("a")
    assert m.num_free_pages() == 3 and m.reserve("b", 16)
    m.check_invariants()
    with pytest.raises(CacheError, match="released twice"):
        m.release("a")
    with pytest.raises(CacheError, match="already admitted"):
        m.admit("b")
    with pytest.raises(CacheError, match="at most"):
        m.reserve("b", 65)


def test_slots_run_out_and_come_back():
    m = _manager(seqs=2)
    assert m.admit("a") is not None and m.admit("b") is not None
    assert m.admit("c") is None
    m.release("a")
    assert m.admit("c") is not None
    m.check_invariants()


def test_dirty_and_fresh_slots_are_reported():
    m = _manager()
    slot = m.admit("a")
    assert m.fresh_slots == {slot}
    m.reserve("a", 5)
    assert m.dirty_slots == {slot}
    m.dirty_slots.clear()
    m.reserve("a", 6)  # no new page: the device copy is still right
    assert not m.dirty_slots
    m.release("a")
    assert m.dirty_slots == {slot}


def test_window_group_gives_pages_back_as_it_moves():
    m = _manager(num_pages=12, page=4, windows=(0, 6))
    m.admit("a")
    assert m.reserve("a", 20)
    assert len(m.pages_of("a", 0)) == 5 and len(m.pages_of("a", 1)) == 5
    # the next query is at position 20 and reads [15, 20]: pages 0..2 (positions < 12) are dead
    assert m.trim("a", 20) == 3
    assert len(m.pages_of("a", 0)) == 5 and len(m.pages_of("a", 1)) == 2
    assert list(m.tables[1][m.slot_of("a")][:5]) [:3] == [NULL_PAGE] * 3
    m.check_invariants()
    # growing on: only the window group's new page is needed, trimmed ones stay null
    assert m.pages_needed("a", 24, 20) == {0: 1, 1: 1}
    assert m.reserve("a", 24, 20)
    assert m.trim("a", 24) == 1
    m.check_invariants()
    m.release("a")
    assert m.num_free_pages(0) == 11 and m.num_free_pages(1) == 11


def test_window_prompt_longer_than_the_pool_can_run_in_portions():
    """A windowed group needs only the pages a portion's queries can read."""
    m = _manager(num_pages=6, page=4, max_len=256, windows=(8,))  # 5 usable pages = 20 positions
    m.admit("a")
    done = 0
    while done < 200:
        upto = done + 6
        assert m.reserve("a", upto, done), done
        done = upto
        m.trim("a", done)
        m.check_invariants()
    m.release("a")
    assert m.num_free_pages() == 5


@pytest.mark.parametrize("windows", [(0,), (0, 10), (7,)])
@pytest.mark.parametrize("seed", [0, 1, 2, 3])
def test_no_page_lost_or_held_twice_under_random_orders(windows, seed):
    rng = random.Random(seed)
    m = _manager(num_pages=14, page=4, seqs=4, max_len=80, windows=windows)
    live: dict[str, int] = {}
    counter = 0
    for _ in range(600):
        action = rng.random()
        if action < 0.25 and m.num_free_slots:
            rid = f"r{counter}"
            counter += 1
            assert m.admit(rid) is not None
            live[rid] = 0
        elif action < 0.8 and live:
            rid = rng.choice(list(live))
            upto = min(80, live[rid] + rng.choice((1, 1, 1, 2, 5, 9, 17)))
            if upto > live[rid]:
                free_before = {g.group_id: m.num_free_pages(g.group_id) for g in m.groups}
                if m.reserve(rid, upto, live[rid]):
                    live[rid] = upto
                    m.trim(rid, upto)
                else:
                    assert free_before == {g.group_id: m.num_free_pages(g.group_id) for g in m.groups}
        elif live:
            rid = rng.choice(list(live))
            m.release(rid)
            del live[rid]
        m.check_invariants()
        assert sorted(m.live_requests()) == sorted(live)
    for rid in list(live):
        m.release(rid)
    m.check_invariants()
    for g in m.groups:
        assert m.num_free_pages(g.group_id) == 13
    assert m.num_free_slots == 4


def test_layers_are_grouped_by_what_they_keep():
    kv = lambda w, share=None: CacheNeed.keys_and_values(2, 16, window=w, share_with=share)
    needs = [kv(0), kv(16), kv(0), CacheNeed("state", state_shape=(4,)), kv(16), kv(0, share=0)]
    groups, group_of = plan_groups(needs)
    assert [(g.window, g.layers) for g in groups] == [(0, (0, 2, 5)), (16, (1, 4))]
    assert group_of == [0, 1, 0, None, 1, 0]
    with pytest.raises(ValueError, match="owns none"):
        plan_groups([kv(0, share=1), CacheNeed("none")])
    with pytest.raises(ValueError, match="same positions"):
        plan_groups([kv(0), kv(8, share=0)])


def test_a_mixer_names_its_paged_tensors_and_their_layout():
    """What a page holds is the mixer's to say: keys and values of different widths, or one
    latent row per token without values; the bytes a page id costs are summed from what is named."""
    from rapid_llm_amd.cache.storage import page_bytes
    from rapid_llm_amd.parts import PagedSpec

    attention = CacheNeed.keys_and_values(2, 16)
    assert [(p.name, p.page_shape(10, 4)) for p in attention.paged] == [("k", (10, 2, 4, 16)), ("v", (10, 2, 16, 4))]
    latent = CacheNeed("paged", paged=(PagedSpec("latent", (24,), 0),))
    assert latent.paged[0].page_shape(10, 4) == (10, 4, 24)
    uneven = CacheNeed("paged", window=8, paged=(PagedSpec("k", (3, 32), 1), PagedSpec("v", (3, 8), 1, "float32")))
    needs = [attention, latent, uneven, CacheNeed("state", state_shape=(4,))]
    groups, group_of = plan_groups(needs)
    assert group_of == [0, 0, 1, None]
    # a page of 4 positions, 2-byte elements: (2*16 + 2*16) + 24 elements in group 0;
    # 3*32 two-byte and 3*8 four-byte elements in group 1
    assert page_bytes(needs, group_of, 4, 2) == {0: 4 * 2 * (64 + 24), 1: 4 * (96 * 2 + 24 * 4)}
    with pytest.raises(ValueError, match="names 0 paged tensors"):
        CacheNeed("paged")
    with pytest.raises(ValueError, match="names 1 paged tensors"):
        CacheNeed("state", paged=(PagedSpec("x", (2,)),))
    with pytest.raises(ValueError, match="alike"):
        CacheNeed("paged", paged=(PagedSpec("k", (2,)), PagedSpec("k", (3,))))
    with pytest.raises(ValueError, match="slot_axis"):
        PagedSpec("k", (2, 4), 3)
    with pytest.raises(ValueError, match="other paged tensors"):
        plan_groups([attention, CacheNeed.keys_and_values(2, 32, share_with=0)])
