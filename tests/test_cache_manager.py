"""The page bookkeeping without a GPU: no page is lost, held twice or freed twice, under fixed
vectors and under random orders of requests (the reference's idiom:
tests/gpu_page_table_tests.cpp:98-178 vectors, 226-285 random run against a set oracle)."""
import random

import pytest

from mini_llm_runtime_amd.cache import CacheError, CacheFull, PageBook


def book(pages=8, page=16, slots=4, max_length=256, window=None):
    b = PageBook(slots, max_length)
    b.add_group(page, pages, window)
    return b


def mapped(b, slot, group=0):
    return [p for p in b.table(group)[slot].tolist() if p >= 0]


def test_page_edges():
    b = book(pages=8, page=16)
    s = b.acquire_slot()
    total = 0
    for target, pages in [(1, 1), (15, 1), (16, 1), (17, 2), (31, 2), (32, 2), (33, 3), (64, 4), (65, 5)]:
        b.commit([s], [target - total])
        total = target
        assert b.length(s) == target and len(mapped(b, s)) == pages and b.free_pages() == 8 - pages
        b.check()
    b.release_slot(s)
    assert b.free_pages() == 8 and mapped(b, s) == []
    b.check()


def test_exhaustion_changes_nothing():
    b = book(pages=4, page=16)
    s0, s1 = b.acquire_slot(), b.acquire_slot()
    b.commit([s0], [40])                        # 3 pages
    before = (b.table().copy(), b.free_pages(), b.length(s0), b.length(s1))
    with pytest.raises(CacheFull, match="needs 2 more pages but only 1"):
        b.prepare([s0, s1], [8, 17])            # s0 fits in its tail page; s1 needs 2
    with pytest.raises(CacheFull):
        b.commit([s0, s1], [8, 17])
    assert (b.table() == before[0]).all() and (b.free_pages(), b.length(s0), b.length(s1)) == before[1:]
    b.commit([s0, s1], [8, 16])                 # exactly the last page
    assert b.free_pages() == 0
    b.check()


def test_freed_pages_are_used_again_at_once():
    b = book(pages=4, page=8)
    s0 = b.acquire_slot()
    b.commit([s0], [20])
    held = mapped(b, s0)
    b.release_slot(s0)
    s1 = b.acquire_slot()
    b.commit([s1], [8])
    assert mapped(b, s1)[0] == held[-1]         # LIFO: the page freed last comes first
    b.check()


def test_refused_batches():
    b = book(pages=8, page=16, slots=2, max_length=64)
    s = b.acquire_slot()
    for slots, counts in [([3], [1]), ([-1], [1]), ([1], [1]), ([s], [0]), ([s], [-2]), ([s, s], [1, 1]), ([s], [65])]:
        with pytest.raises(CacheError):
            b.prepare(slots, counts)
    b.commit([s], [64])
    with pytest.raises(CacheError, match="max_length"):
        b.prepare([s], [1])
    assert b.length(s) == 64
    b.check()


def test_slots_run_out_and_double_free():
    b = book(slots=2)
    s0, s1 = b.acquire_slot(), b.acquire_slot()
    assert {s0, s1} == {0, 1} and b.free_slots() == 0
    with pytest.raises(CacheFull):
        b.acquire_slot()
    b.release_slot(s0)
    with pytest.raises(CacheError, match="not live"):
        b.release_slot(s0)
    with pytest.raises(CacheError):
        b.length(s0)
    assert b.acquire_slot() == s0
    b.check()


def test_window_gives_pages_back_when_passed():
    b = book(pages=6, page=4, max_length=1000, window=6)
    s = b.acquire_slot()
    length = 0
    for n in [3, 5, 1, 1, 1, 7, 2, 1, 1, 1, 1, 9]:
        b.commit([s], [n])
        length += n
        # the step's own queries may look back a window from its first token: nothing is retired before it ran
        b.retire([s])
        row = b.table()[s]
        first_needed = max(0, length - 6 + 1)
        for blk in range((length + 3) // 4):
            if (blk + 1) * 4 <= first_needed:
                assert row[blk] == -1, (length, blk)
            else:
                assert row[blk] >= 0, (length, blk)
        assert b.free_pages() == 6 - sum(1 for p in row if p >= 0)
        b.check()
    b.release_slot(s)
    assert b.free_pages() == 6
    b.check()


def test_two_groups_with_different_needs():
    b = PageBook(3, 512)
    full = b.add_group(16, 10, None)
    win = b.add_group(16, 4, 20)
    s = b.acquire_slot()
    b.commit([s], [60])
    assert len(mapped(b, s, full)) == 4 and len(mapped(b, s, win)) == 4
    b.retire([s])
    assert len(mapped(b, s, full)) == 4 and len(mapped(b, s, win)) == 2       # keys < 41 are out of sight
    b.commit([s], [30])                                                          # 2 more pages in each group
    with pytest.raises(CacheFull, match="group 1"):
        b.prepare([s], [30])                                                     # the window pool is the short one
    b.retire([s])
    b.commit([s], [30])
    b.check()


def test_dirty_rows():
    b = book(pages=8, page=16, slots=3)
    assert b.take_dirty() == [0, 1, 2]
    s0, s1 = b.acquire_slot(), b.acquire_slot()
    b.commit([s0], [5])
    assert b.take_dirty() == [s0]
    b.commit([s0, s1], [3, 1])
    assert b.take_dirty() == [s1]              # s0 stayed inside its page
    b.release_slot(s0)
    assert b.take_dirty() == [s0]


@pytest.mark.parametrize("seed,window", [(0, None), (1, None), (2, 24), (3, 7)])
def test_random_orders_of_requests(seed, window):
    rng = random.Random(seed)
    page, pages, slots, max_length = 8, 24, 5, 120
    b = PageBook(slots, max_length)
    b.add_group(page, pages, window)
    live = {}                                   # slot -> length (the oracle)
    retired = {}                                # slot -> first block still held
    for _ in range(6000):
        op = rng.random()
        if op < 0.15 and len(live) < slots:
            s = b.acquire_slot()
            assert s not in live
            live[s], retired[s] = 0, 0
        elif op < 0.25 and live:
            s = rng.choice(sorted(live))
            b.release_slot(s)
            del live[s], retired[s]
        elif live:
            chosen = rng.sample(sorted(live), rng.randint(1, len(live)))
            counts = [rng.choice([1, 1, 1, 2, 5, 9, 17]) for _ in chosen]
            need = 0
            too_long = False
            for s, n in zip(chosen, counts):
                too_long |= live[s] + n > max_length
                need += -(-(live[s] + n) // page) - (-(-live[s] // page))
            held = sum(-(-live[s] // page) - retired[s] for s in live)
            free = pages - held
            assert b.free_pages() == free
            try:
                b.commit(chosen, counts)
                ok = True
            except CacheFull:
                ok = False
                assert not too_long and need > free
            except CacheError:
                ok = False
                assert too_long
            if ok:
                assert not too_long and need <= free
                for s, n in zip(chosen, counts):
                    live[s] += n
                b.retire(chosen)
                if window:
                    for s in chosen:
                        retired[s] = max(retired[s], max(0, live[s] - window + 1) // page)
        b.check()
        # the same page is never in two rows, and every row holds exactly the blocks it needs
        seen = set()
        for s in live:
            row = b.table()[s].tolist()
            blocks = -(-live[s] // page)
            for blk, p in enumerate(row):
                if retired[s] <= blk < blocks:
                    assert p >= 0 and p not in seen
                    seen.add(p)
                else:
                    assert p == -1
        assert len(seen) + b.free_pages() == pages


def test_commit_reports_first_positions():
    b = book(pages=8, page=16, slots=3)
    s0, s1 = b.acquire_slot(), b.acquire_slot()
    assert b.commit_first([s0, s1], [5, 20]) == [0, 0]
    assert b.commit_first([s1, s0], [1, 3]) == [20, 5]
    before = (b.table().copy(), b.free_pages(), b.length(s0), b.length(s1))
    with pytest.raises(CacheFull):
        b.commit_first([s0, s1], [60, 60])
    with pytest.raises(CacheError):
        b.commit_first([s0, 2], [1, 1])
    assert (b.table() == before[0]).all() and (b.free_pages(), b.length(s0), b.length(s1)) == before[1:]
    b.check()


def test_a_spec_names_what_a_page_holds_and_groups_have_page_sizes_of_their_own():
    """What is allocated follows from the specs alone: every tensor of a spec as [entries, pages + 1, *shape
    within a page], pages of the group's own size and element type; equal specs share a group.  (On the CPU:
    the manager's memory is ordinary tensors there.)"""
    import torch

    from mini_llm_runtime_amd.cache import PAGE, CacheManager, KvSpec, PagedSpec, StateSpec
    latent = PagedSpec((("latent", (PAGE, 6)), ("gate", (3, PAGE))), page_size=4, dtype=torch.float32)
    specs = [KvSpec(2, 16), latent, KvSpec(2, 16), StateSpec((5,), torch.float32), KvSpec(2, 16, window=24), None, latent]
    m = CacheManager(specs, torch.bfloat16, "cpu", page_size=16, max_tokens=100, max_slots=3, max_length=64)
    assert m.group_page_size == [16, 4, 16] and m.group_pages == [7, 25, 7]
    assert m.kv_view(0).k_pages.shape == (8, 2, 16, 16) and m.kv_view(2).v_pages.shape == (8, 2, 16, 16)
    assert m.kv_view(0).group == m.kv_view(2).group != m.kv_view(4).group
    first, second = m.paged_view(1), m.paged_view(6)
    assert first.group == second.group and first.page_size == 4 and first.window is None
    assert first.tensors["latent"].shape == (26, 4, 6) and first.tensors["gate"].shape == (26, 3, 4)
    assert first.tensors["latent"].dtype == torch.float32 and m.kv_view(0).k_pages.dtype == torch.bfloat16
    assert first.tensors["latent"].data_ptr() != second.tensors["latent"].data_ptr()
    assert first.block_table.shape == (4, 16) and m.kv_view(0).block_table.shape == (4, 4)
    assert torch.isnan(first.tensors["latent"]).all()                  # a never-written page shows
    planned = CacheManager.plan(specs, torch.bfloat16, 16, 100, 3, 64)
    assert planned == (m.kv_bytes(), m.table_bytes(), m.state_bytes())
    assert m.kv_bytes() == 3 * 8 * 2 * (2 * 16 * 16) * 2 + 2 * 26 * (4 * 6 + 3 * 4) * 4
    assert m.reserve_unit() == 16
    # a request takes pages of every group, each in its own size, and gives them all back
    slot = m.acquire_slot()
    m.prepare([slot], [21])
    m.commit([slot], [21])
    assert [m.group_pages[g] - m.free_pages(g) for g in range(3)] == [2, 6, 2]
    m.release_slot(slot)
    assert [m.free_pages(g) for g in range(3)] == m.group_pages
    m.check()
    odd = CacheManager([KvSpec(1, 16), PagedSpec((("x", (PAGE,)),), page_size=24)], torch.float32, "cpu", 16, 96, 2, 96)
    assert odd.reserve_unit() == 48


@pytest.mark.parametrize("seed", range(6))
def test_the_largest_pool_that_fits_a_budget(seed):
    """`CacheManager.tokens_that_fit`: a multiple of every group's page size, within the budget by the manager's
    own plan, one unit more would not be (unless the slots cannot hold more), and nothing when not one unit fits."""
    import math
    import torch
    from mini_llm_runtime_amd.cache import CacheManager, KvSpec, PagedSpec, StateSpec, PAGE
    rng = random.Random(seed)
    specs = [KvSpec(rng.randint(1, 4), rng.choice([16, 32, 64]), None) for _ in range(rng.randint(1, 3))]
    if rng.random() < 0.5:
        specs.append(KvSpec(2, 16, rng.choice([8, 24])))                         # a windowed group of its own
    if rng.random() < 0.5:
        specs.append(PagedSpec((("latent", (PAGE, 6)),), page_size=rng.choice([4, 12]), dtype=torch.float32))
    if rng.random() < 0.5:
        specs.append(StateSpec((rng.randint(1, 40),), torch.float32))
    rng.shuffle(specs)
    page, slots, length = rng.choice([8, 16, 32]), rng.randint(1, 9), rng.randint(10, 500)
    unit = 1
    for s in specs:
        size = getattr(s, "page_size", None) or (page if not isinstance(s, StateSpec) else 1)
        unit = unit * size // math.gcd(unit, size)
    total = lambda tokens: sum(CacheManager.plan(specs, torch.bfloat16, page, tokens, slots, length))
    most = slots * -(-length // unit) * unit
    for budget in (total(most) + 5, total(most) - 1, total(3 * unit), total(unit) + 1, total(unit) - 1, 0):
        got = CacheManager.tokens_that_fit(specs, torch.bfloat16, page, slots, length, budget)
        assert got % unit == 0 and 0 <= got <= most
        if got:
            assert total(got) <= budget
            assert got == most or total(got + unit) > budget
        else:
            assert total(unit) > budget
