"""The cache manager's bookkeeping (CPU): no page lost, held twice or freed twice, under random
orders of requests; windows give pages back; slots.  Vectors marked (ref) restate
reference: torchllms/models/test_paged_kv.py:53-136,303-426."""

import random

import pytest
import torch

from torchllms_amd.cache import CacheGroupSpec, CacheManager, OutOfPages, OutOfSlots, PagePool, StateSlotSpec, group_layers
from torchllms_amd.parts import KVNeed, StateNeed


def mk(num_pages=16, page_size=4, max_seqs=4, window=0, device=None, states=()):
    groups = [CacheGroupSpec("kv0", (0, 1, 2), num_kv_heads=2, head_dim=8, window=window)]
    return CacheManager(groups, list(states), page_size, num_pages, max_seqs, device=device)


def test_fresh_pool_is_all_free():  # (ref)
    c = mk()
    assert c.live == [] and c.free_pages() == 16 and c.free_slots == 4
    c.check_invariants()


def test_admit_takes_no_pages_and_pages_follow_ceil_division():  # (ref: 1->1, 4->1, 5->2, 13->4 at P=4)
    c = mk()
    c.admit("r")
    assert c.free_pages() == 16
    for total, pages in [(1, 1), (4, 1), (5, 2), (13, 4)]:
        n = total - c.num_tokens("r")
        c.extend("r", n)
        c.advance("r", n)
        assert len(c.block_table("r")) == pages and c.free_pages() == 16 - pages
        c.check_invariants()


def test_free_returns_everything_and_pages_are_used_again():  # (ref)
    c = mk()
    c.admit("a")
    c.extend("a", 13)
    c.advance("a", 13)
    first = list(c.block_table("a"))
    c.free("a")
    assert c.free_pages() == 16 and c.free_slots == 4
    c.admit("b")
    c.extend("b", 8)
    assert set(c.block_table("b")) <= set(first)  # recently freed pages are handed out again
    c.check_invariants()
    with pytest.raises(KeyError, match="freed twice"):
        c.free("a")


def test_out_of_pages_is_all_or_nothing():  # (ref: raises; here nothing stays attached)
    c = mk(num_pages=2)
    c.admit("a")
    c.extend("a", 8)
    c.admit("b")
    assert not c.can_extend("b", 1)
    with pytest.raises(OutOfPages):
        c.extend("b", 1)
    assert c.block_table("b") == [] and c.free_pages() == 0
    c.check_invariants()
    c.free("a")
    assert c.can_extend("b", 8)
    c.extend("b", 5)
    c.check_invariants()


def test_double_release_and_sharing():  # (ref: refcounts)
    p = PagePool(4)
    pages = p.take(2)
    p.share(pages)
    p.give_back(pages)
    assert p.free_count == 2
    p.give_back(pages)
    assert p.free_count == 4
    with pytest.raises(RuntimeError, match="released twice"):
        p.give_back(pages[:1])
    with pytest.raises(OutOfPages):
        p.take(5)


def test_slots_are_recycled_and_bounded():
    c = mk(max_seqs=2)
    s0, s1 = c.admit("a"), c.admit("b")
    assert {s0, s1} == {0, 1}
    with pytest.raises(OutOfSlots):
        c.admit("c")
    with pytest.raises(ValueError, match="already live"):
        c.admit("a")
    c.free("a")
    assert c.admit("c") == s0
    c.check_invariants()


def test_advance_needs_pages():
    c = mk()
    c.admit("a")
    with pytest.raises(RuntimeError, match="extend first"):
        c.advance("a", 1)


def test_truncate_gives_trailing_pages_back():
    c = mk()
    c.admit("a")
    c.extend("a", 13)
    c.advance("a", 13)
    c.truncate("a", 5)
    assert c.num_tokens("a") == 5 and len(c.block_table("a")) == 2 and c.free_pages() == 14
    c.check_invariants()


def test_window_gives_pages_back_once_passed():
    c = mk(num_pages=6, page_size=4, window=6)
    c.admit("a")
    for step in range(40):  # 40 tokens, one at a time, in a pool of 24 token places
        c.extend("a", 1)
        c.advance("a", 1)
        c.check_invariants()
        n = c.num_tokens("a")
        bt = c.block_table("a")
        lo = max(n - 6 + 1, 0)  # the next query (position n) reads from here on
        for b, page in enumerate(bt):
            if (b + 1) * 4 <= lo:
                assert page == -1
            else:
                assert page >= 0
        assert sum(p >= 0 for p in bt) <= 3
    c.free("a")
    assert c.free_pages() == 6


def test_window_keeps_what_a_portion_needs():
    c = mk(num_pages=8, page_size=4, window=5)
    c.admit("a")
    c.extend("a", 9)
    c.advance("a", 9)  # next query at 9 reads 5..9 -> block 0 (0..3) is passed
    assert c.block_table("a")[0] == -1 and c.block_table("a")[1] >= 0
    c.extend("a", 7)  # portion 9..15: query 9 still needs 5.., so nothing more may go before the step
    assert c.block_table("a")[1] >= 0
    c.advance("a", 7)  # next query at 16 reads 12..16
    assert c.block_table("a")[:3] == [-1, -1, -1] and c.block_table("a")[3] >= 0
    c.check_invariants()


def test_groups_are_formed_by_need():
    needs = [
        (0, KVNeed(2, 16, 0)), (1, KVNeed(2, 16, 128)), (2, KVNeed(2, 16, 0)), (3, StateNeed((4, 8))),
        (4, None), (5, KVNeed(2, 16, 128)), (6, StateNeed((4, 8))),
    ]
    groups, states = group_layers(needs)
    assert [(g.run_ids, g.window) for g in groups] == [((0, 2), 0), ((1, 5), 128)]
    assert [(s.run_ids, s.shape) for s in states] == [((3, 6), (4, 8))]


def test_two_groups_have_pages_of_their_own():
    groups = [CacheGroupSpec("full", (0,), 2, 8, 0), CacheGroupSpec("win", (1,), 2, 8, 4)]
    c = CacheManager(groups, [], page_size=4, num_pages={"full": 8, "win": 3}, max_seqs=2)
    c.admit("a")
    for _ in range(30):
        c.extend("a", 1)
        c.advance("a", 1)
        c.check_invariants()
    assert c.free_pages(0) == 0 and sum(p >= 0 for p in c.block_table("a", 1)) <= 2
    assert not c.can_extend("a", 3)  # the full group is exhausted, although the window group is not
    assert c.pages_short("a", 3) == {0: 1, 1: 0}


def test_state_slots_are_zeroed_on_admission():
    st = [StateSlotSpec("s", (0, 1), (3,), "float32")]
    c = mk(max_seqs=2, device="cpu", states=st)
    assert c.state_tensors[0].shape == (2, 2, 3)
    slot = c.admit("a")
    c.state_view(1).tensor[slot] += 5
    assert c.state_tensors[0][1, slot].tolist() == [5, 5, 5]
    c.free("a")
    assert c.admit("b") == slot
    assert c.state_tensors[0][:, slot].abs().sum() == 0


def test_kv_views_and_gather_on_cpu_tensors():
    c = mk(device="cpu")
    assert c.k_pages[0].shape == (3, 16, 2, 4, 8)
    v = c.kv_view(1)
    assert v.k_pages.shape == (16, 2, 4, 8) and v.group == 0 and v.writes
    assert not c.view_for_run(2, cache_from=1).writes
    c.admit("a")
    c.extend("a", 6)
    c.advance("a", 6)
    bt = c.block_table("a")
    for pos in range(6):
        c.k_pages[0][1, bt[pos // 4], :, pos % 4] = pos + 1
    k, _ = c.gather_kv("a", 1)
    assert k[:, 0, 0].tolist() == [1, 2, 3, 4, 5, 6]


@pytest.mark.parametrize("seed", range(6))
def test_random_orders_keep_the_invariants(seed):
    rng = random.Random(seed)
    window = rng.choice([0, 0, 5, 11])
    c = mk(num_pages=rng.choice([6, 12, 30]), page_size=rng.choice([2, 4, 8]), max_seqs=4, window=window)
    live = {}
    next_id = 0
    for _ in range(600):
        op = rng.random()
        if op < 0.2 and c.free_slots:
            c.admit(next_id)
            live[next_id] = 0
            next_id += 1
        elif op < 0.85 and live:
            rid = rng.choice(list(live))
            n = rng.choice([1, 1, 1, 2, 3, 7, 16])
            if c.can_extend(rid, n):
                before = c.free_pages()
                c.extend(rid, n)
                c.advance(rid, n)
                live[rid] += n
                assert c.num_tokens(rid) == live[rid]
                assert before - c.free_pages() <= -(-n // c.page_size) + 1
            else:
                held = list(c.block_table(rid))
                with pytest.raises(OutOfPages):
                    c.extend(rid, n)
                assert c.block_table(rid) == held
        elif live:
            rid = rng.choice(list(live))
            c.free(rid)
            del live[rid]
        c.check_invariants()
    for rid in list(live):
        c.free(rid)
    c.check_invariants()
    assert c.free_pages() == c.pools[0].num_pages and c.free_slots == 4


def test_groups_differ_in_page_size_and_element_type():
    """Needs that name a page size or an element type of their own form groups of their own, whose
    tables, pools and tensors follow their own sizes."""
    needs = [
        ((0, "mixer"), KVNeed(2, 8, 0)), ((1, "mixer"), KVNeed(2, 8, 0, page_size=8)),
        ((2, "mixer"), KVNeed(2, 8, 0)), ((3, "mixer"), KVNeed(2, 8, 0, page_size=8, dtype="float32")),
    ]
    groups, _ = group_layers(needs)
    assert [(g.run_ids, g.page_size, g.dtype) for g in groups] == [
        (((0, "mixer"), (2, "mixer")), 0, None), (((1, "mixer"),), 8, None), (((3, "mixer"),), 8, "float32"),
    ]
    pages = CacheManager.pages_for_tokens(groups, 4, 40)
    assert pages == {"kv0": 10, "kv1": 5, "kv2": 5}
    assert CacheManager.bytes_per_token(groups, torch.bfloat16) == 2 * 2 * 8 * (2 * 2 + 1 * 2 + 1 * 4)
    c = CacheManager(groups, [], page_size=4, num_pages=pages, max_seqs=2, dtype=torch.bfloat16, device="cpu")
    assert c.page_sizes == [4, 8, 8]
    assert c.k_pages[0].shape == (2, 10, 2, 4, 8) and c.k_pages[1].shape == (1, 5, 2, 8, 8)
    assert c.k_pages[1].dtype == torch.bfloat16 and c.k_pages[2].dtype == torch.float32
    assert c.view((1, "mixer")).page_size == 8 and c.view((0, "mixer")).page_size == 4
    c.admit("a")
    assert c.new_pages_needed("a", 9) == [3, 2, 2]
    c.extend("a", 9)
    c.advance("a", 9)
    assert [len(c.block_table("a", g)) for g in range(3)] == [3, 2, 2]
    assert c.new_pages_needed("a", 3) == [0, 0, 0] and c.new_pages_needed("a", 4) == [1, 0, 0]
    assert c.new_pages_needed("a", 8) == [2, 1, 1]
    c.truncate("a", 8)
    assert [len(c.block_table("a", g)) for g in range(3)] == [2, 1, 1]
    # the small pages end first: 40 tokens fill all three pools, one more fits none
    c.extend("a", 32)
    c.advance("a", 32)
    assert [c.free_pages(g) for g in range(3)] == [0, 0, 0] and not c.can_extend("a", 1)
    c.check_invariants()
    c.free("a")
    assert [c.free_pages(g) for g in range(3)] == [10, 5, 5]


@pytest.mark.parametrize("seed", range(6))
def test_random_orders_keep_the_invariants_with_mixed_page_sizes(seed):
    rng = random.Random(100 + seed)
    sizes = [rng.choice([2, 4, 8]), rng.choice([3, 16]), rng.choice([4, 5])]
    windows = [0, rng.choice([0, 7]), 0]
    groups = [CacheGroupSpec(f"kv{g}", (g,), 1, 4, windows[g], page_size=p) for g, p in enumerate(sizes)]
    tokens = rng.choice([40, 90])
    c = CacheManager(groups, [], 4, CacheManager.pages_for_tokens(groups, 4, tokens), max_seqs=3)
    live = {}
    next_id = 0
    for _ in range(500):
        op = rng.random()
        if op < 0.2 and c.free_slots:
            c.admit(next_id)
            live[next_id] = 0
            next_id += 1
        elif op < 0.85 and live:
            rid = rng.choice(list(live))
            n = rng.choice([1, 1, 1, 2, 3, 7, 16])
            need = c.new_pages_needed(rid, n)
            if c.can_extend(rid, n):
                before = [c.free_pages(g) for g in range(3)]
                c.extend(rid, n)
                assert [b - c.free_pages(g) for g, b in enumerate(before)] == need
                c.advance(rid, n)
                live[rid] += n
            else:
                held = [list(c.block_table(rid, g)) for g in range(3)]
                with pytest.raises(OutOfPages):
                    c.extend(rid, n)
                assert [c.block_table(rid, g) for g in range(3)] == held
        elif live:
            rid = rng.choice(list(live))
            c.free(rid)
            del live[rid]
        c.check_invariants()
    for rid in list(live):
        c.free(rid)
    c.check_invariants()
    assert all(c.free_pages(g) == c.pools[g].num_pages for g in range(3))
