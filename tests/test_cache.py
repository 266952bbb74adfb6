"""The allocator and the cache manager (CPU): no page lost, held twice or freed twice,
under random orders of requests; windows give pages back; rows move without moving pages."""

import random

import pytest
import torch

from socrates_amd.cache import BlockAllocator, CacheManager, OutOfBlocks, blocks_for
from socrates_amd.parts import PagedKV, RowState


def test_blocks_for_reference_vector():
    # tests/test_paging.py:6-10 of the reference
    for tokens, blocks in [(0, 0), (1, 1), (15, 1), (16, 1), (17, 2), (2047, 128), (2048, 128), (2049, 129)]:
        assert blocks_for(tokens, 16) == blocks


def test_allocator_semantics():
    a = BlockAllocator(10)
    assert a.alloc(10) == list(range(1, 11)) and a.n_free == 0        # first allocation is 1..10
    a.free(list(range(1, 11)))
    assert a.n_free == 10
    with pytest.raises(ValueError):
        a.free([0])                                                    # the null page
    got = a.alloc(4)
    with pytest.raises(OutOfBlocks):
        a.alloc(7)
    assert a.n_free == 6                                               # a failed alloc changes nothing
    with pytest.raises(ValueError):
        a.free([got[0], got[0]])                                       # duplicate in one call
    with pytest.raises(ValueError):
        a.free([got[1], 9])                                            # 9 is not held: nothing is freed
    assert a.n_free == 6 and all(a.is_held(p) for p in got)
    a.free(got[:2])
    with pytest.raises(ValueError):
        a.free(got[:1])                                                # double free
    assert a.alloc(2) == got[:2]                                       # freed last, handed out first
    with pytest.raises(ValueError):
        BlockAllocator(0)


def manager(needs=None, rows=4, max_len=128, bs=8, pages=20):
    return CacheManager(needs or [PagedKV(2, 16)] * 2, rows, max_len, bs, pages, torch.float32, "cpu")


def test_pages_are_taken_lazily_and_returned():
    c = manager()
    r = c.open_row()
    c.reserve(r, 9)
    assert c.held_pages(r) == [2] and c.n_free_pages == 18
    c.advance(r, 9)
    c.reserve(r, 16)                                                   # still two pages
    assert c.held_pages(r) == [2]
    c.reserve(r, 17)
    assert c.held_pages(r) == [3]
    c.sync()
    table = c.slot(0).block_table
    assert table[r, :3].tolist() == [1, 2, 3] and table[r, 3:].abs().sum() == 0
    assert c.slot(0).block_table is c.slot(1).block_table              # one table per group
    assert c.slot(0).k.shape == (21, 2, 8, 16) and c.slot(0).k is not c.slot(1).k
    c.close_row(r)
    c.sync()
    assert c.n_free_pages == 20 and table.abs().sum() == 0 and c.check()
    with pytest.raises(ValueError):
        c.close_row(r)                                                 # not open any more


def test_out_of_blocks_takes_nothing():
    c = manager(pages=4)
    a, b = c.open_row(), c.open_row()
    c.reserve(a, 24)
    with pytest.raises(OutOfBlocks):
        c.reserve(b, 17)                                               # needs 3, 1 free
    assert c.held_pages(b) == [0] and c.n_free_pages == 1 and c.check()
    assert c.pages_short(b, 17) == 2 and c.pages_short(b, 8) == 0
    with pytest.raises(ValueError):
        c.reserve(a, 129)                                              # beyond max_len


def test_window_group_gives_pages_back_as_the_window_passes():
    full, win = PagedKV(2, 16), PagedKV(2, 16, window=10)
    c = manager([full, win, full, win], pages=12)
    assert len(c.groups) == 2
    r = c.open_row()
    for step_len in (13, 1, 1, 20, 1, 7):
        c.reserve(r, c.length(r) + step_len)
        c.advance(r, step_len)
        c.check()
    n = c.length(r)
    held_full, held_win = c.held_pages(r)
    assert held_full == blocks_for(n, 8)
    # the next token sits at position n and sees keys n-9..n: pages before (n-9)//8 are gone
    c.reserve(r, n + 1)
    assert c.groups[1].first_live[r] == (n - 9) // 8
    assert c.held_pages(r)[1] == blocks_for(n + 1, 8) - (n - 9) // 8
    win_table = c.groups[1].host_table[r]
    assert not win_table[:c.groups[1].first_live[r]].any()             # dropped entries point at the null page
    c.close_row(r)
    assert c.free_pages() == [12, 12] and c.check()


def test_move_row_moves_table_and_state_not_pages():
    c = manager([PagedKV(2, 16), RowState((3, 5))])
    a = c.open_row()
    c.reserve(a, 20)
    c.advance(a, 20)
    c.scalars.temperature[a], c.scalars.seed[a], c.scalars.draws[a] = 0.7, 99, 4
    c.slot(1).state[a] = 2.5
    c.slot(0).k[1:4] = 1.0
    before = c.slot(0).k.clone()
    ptr = c.slot(0).k.data_ptr()
    held = c.groups[0].held_by(a)
    c.move_row(a, 3)
    assert c.groups[0].held_by(3) == held and c.groups[0].held_by(a) == []
    assert c.length(3) == 20 and c.length(a) == 0
    assert (c.scalars.temperature[3], c.scalars.seed[3], c.scalars.draws[3]) == (pytest.approx(0.7), 99, 4)
    assert c.slot(1).state[3].eq(2.5).all()
    assert c.slot(0).k.data_ptr() == ptr and torch.equal(c.slot(0).k, before)   # no page moved
    assert c.open_rows == [3] and c.check()
    again = c.open_row()
    assert again == 0 and c.slot(1).state[0].abs().sum() == 0          # state is cleared when a row opens
    with pytest.raises(ValueError):
        c.move_row(3, 0)                                               # the target is open


@pytest.mark.parametrize("seed", range(6))
def test_random_orders_keep_the_books(seed):
    """Open, grow, trim and close rows in random order, with a windowed group beside a full
    one; after every action no page is lost, held twice, or held by a closed row."""
    rng = random.Random(seed)
    c = manager([PagedKV(1, 16), PagedKV(1, 16, window=rng.choice([5, 16, 40]))], rows=5,
                max_len=160, bs=rng.choice([4, 8, 16]), pages=rng.choice([12, 30]))
    live = []
    for _ in range(400):
        action = rng.random()
        if action < 0.25 and c.n_free_rows:
            live.append(c.open_row())
        elif action < 0.85 and live:
            r = rng.choice(live)
            n = rng.choice([1, 1, 1, 2, 7, 19, 33])
            if c.length(r) + n > c.max_len:
                continue
            free_before, held_before = c.free_pages(), c.held_pages(r)
            try:
                c.reserve(r, c.length(r) + n)
                c.advance(r, n)
            except OutOfBlocks:
                # nothing was taken (pages a window has passed may have been given back)
                assert all(a >= b for a, b in zip(c.free_pages(), free_before))
                assert all(a <= b for a, b in zip(c.held_pages(r), held_before))
        elif live:
            r = live.pop(rng.randrange(len(live)))
            c.close_row(r)
        c.check()
    for r in live:
        c.close_row(r)
    assert all(f == g.allocator.num_blocks for f, g in zip(c.free_pages(), c.groups)) and c.check()
