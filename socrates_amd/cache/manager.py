"""The cache manager: pages, block tables, per-request state.

Layout of one page pool follows the reference's paged cache
(model/qwen/qwen_kv_paged.py:34-74): per cache slot a K and a V pool of shape
[num_blocks + 1, n_kv_heads, block_size, head_dim] (heads before slots, so one
(page, head) is one contiguous tile), page 0 the null page, and one int32 block
table [max_rows, table_width] that all slots of a group share.

Beyond the reference: cache slots are collected into *groups* by what they need
(all keys, or a window of them; a page shape); each group has its own allocator,
table and pools. Pages are taken when a step needs them, not reserved at
admission, and given back when a row closes or, in a windowed group, when every
position of a page lies behind the window of every token still to come. Mixers
with a state of fixed size get a float32 tensor [max_rows, *shape] per slot,
cleared when a row opens. Fixed-size per-request scalars (length, sampling
parameters, counters) live in ``RowScalars``.
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import List, Optional

import numpy as np
import torch

from ..parts.registry import PagedKV, RowState
from .allocator import NULL_PAGE, BlockAllocator, OutOfBlocks, blocks_for
from .staging import PinnedUploader


@dataclass
class PagedSlot:
    """What a paged mixer sees of its cache slot."""
    k: torch.Tensor
    v: torch.Tensor
    block_table: torch.Tensor      # int32 [max_rows, table_width], on the device
    block_size: int
    window: Optional[int]


@dataclass
class StateSlot:
    """What a mixer with fixed-size state sees: float32 [max_rows, *shape]."""
    state: torch.Tensor


class PagedGroup:
    """Cache slots with the same need: one allocator, one table, a pool pair per slot."""

    def __init__(self, need: PagedKV, max_rows, table_width, block_size, num_blocks, dtype, device):
        self.need, self.block_size, self.table_width = need, block_size, table_width
        self.allocator = BlockAllocator(num_blocks)
        # one row more than can be opened: the null row, whose entries all point at the null
        # page, stands in for the padding rows of a fixed-width (captured) decode step
        self.host_table = np.zeros((max_rows + 1, table_width), dtype=np.int32)
        self.table = torch.zeros((max_rows + 1, table_width), dtype=torch.int32, device=device)
        # per row: number of logical blocks ever covered, and the first one still held
        self.covered = [0] * max_rows
        self.first_live = [0] * max_rows
        self.dirty = set()
        self.pool_shape = (num_blocks + 1, need.n_kv_heads, block_size, need.head_dim)
        self.dtype, self.device = dtype, device
        self.pools = {}
        self._upload = PinnedUploader(device) if torch.device(device).type == "cuda" else None

    def add_slot(self, slot_id: int):
        k = torch.zeros(self.pool_shape, dtype=self.dtype, device=self.device)
        v = torch.zeros(self.pool_shape, dtype=self.dtype, device=self.device)
        self.pools[slot_id] = (k, v)

    # -- pages a row needs / can drop ---------------------------------------------------------
    def droppable(self, row: int, next_start: int) -> int:
        """Logical blocks of ``row`` that no token at position >= next_start can see."""
        if self.need.window is None:
            return self.first_live[row]
        first_visible = max(0, next_start - self.need.window + 1)
        return max(self.first_live[row], min(first_visible // self.block_size, self.covered[row]))

    def missing(self, row: int, new_len: int) -> int:
        return max(0, blocks_for(new_len, self.block_size) - self.covered[row])

    def drop_behind(self, row: int, next_start: int):
        upto = self.droppable(row, next_start)
        lo = self.first_live[row]
        if upto > lo:
            pages = [int(p) for p in self.host_table[row, lo:upto]]
            self.allocator.free(pages)
            self.host_table[row, lo:upto] = NULL_PAGE
            self.first_live[row] = upto
            self.dirty.add(row)

    def extend(self, row: int, new_len: int):
        n = self.missing(row, new_len)
        if n:
            lo = self.covered[row]
            if lo + n > self.table_width:
                raise ValueError(f"{new_len} tokens need {lo + n} blocks, the table holds {self.table_width}")
            self.host_table[row, lo:lo + n] = self.allocator.alloc(n)
            self.covered[row] = lo + n
            self.dirty.add(row)

    def release(self, row: int):
        lo, hi = self.first_live[row], self.covered[row]
        if hi > lo:
            self.allocator.free([int(p) for p in self.host_table[row, lo:hi]])
        if hi:
            self.host_table[row, :hi] = NULL_PAGE
            self.dirty.add(row)
        self.covered[row] = self.first_live[row] = 0

    def held_by(self, row: int):
        return [int(p) for p in self.host_table[row, self.first_live[row]:self.covered[row]]]

    def sync(self):
        if self.dirty:
            lo, hi = min(self.dirty), max(self.dirty) + 1
            if self._upload is not None:
                # a snapshot in pinned memory: the host may change its table again before
                # the queued copy runs
                self._upload(self.host_table[lo:hi], into=self.table[lo:hi])
            else:
                self.table[lo:hi].copy_(torch.from_numpy(self.host_table[lo:hi]))
            self.dirty.clear()


class RowScalars:
    """Fixed-size state of each request, by row: how many tokens its cache holds, its
    sampling parameters and its random stream (seed and draws made so far)."""

    def __init__(self, max_rows: int):
        self.length = np.zeros(max_rows, dtype=np.int64)
        self.temperature = np.zeros(max_rows, dtype=np.float32)
        self.seed = np.zeros(max_rows, dtype=np.uint64)
        self.draws = np.zeros(max_rows, dtype=np.int64)

    _FIELDS = ("length", "temperature", "seed", "draws")

    def clear(self, row: int):
        for f in self._FIELDS:
            getattr(self, f)[row] = 0

    def move(self, src: int, dst: int):
        for f in self._FIELDS:
            a = getattr(self, f)
            a[dst], a[src] = a[src], 0


class CacheManager:
    def __init__(self, needs: List[object], max_rows: int, max_len: int, block_size: int,
                 num_blocks: int, dtype, device):
        """needs: per cache slot a PagedKV, a RowState or None (see parts.cache_needs).
        num_blocks: usable pages of every paged group (the null page comes on top)."""
        if block_size < 1 or max_rows < 1 or max_len < 1:
            raise ValueError("block_size, max_rows and max_len must be positive")
        self.max_rows, self.max_len, self.block_size = max_rows, max_len, block_size
        self.dtype, self.device = dtype, device
        self.table_width = blocks_for(max_len, block_size)
        self.groups: List[PagedGroup] = []
        self._slots = []
        by_need = {}
        for slot_id, need in enumerate(needs):
            if isinstance(need, PagedKV):
                group = by_need.get(need)
                if group is None:
                    group = PagedGroup(need, max_rows, self.table_width, block_size, num_blocks,
                                       dtype, device)
                    by_need[need] = group
                    self.groups.append(group)
                group.add_slot(slot_id)
                k, v = group.pools[slot_id]
                self._slots.append(PagedSlot(k, v, group.table, block_size, need.window))
            elif isinstance(need, RowState):
                kinds = {"float32": torch.float32, "int32": torch.int32, "compute": dtype}
                if need.dtype not in kinds:
                    raise ValueError(f"cache slot {slot_id}: a row's state is one of {sorted(kinds)}, not {need.dtype!r}")
                state = torch.zeros((max_rows + 1,) + tuple(need.shape), dtype=kinds[need.dtype], device=device)
                self._slots.append(StateSlot(state))
            elif need is None:
                self._slots.append(None)
            else:
                raise TypeError(f"cache slot {slot_id}: unknown kind of need {need!r}")
        self.scalars = RowScalars(max_rows)
        self._open = [False] * max_rows

    # -- rows ------------------------------------------------------------------------------
    @property
    def open_rows(self):
        return [r for r, o in enumerate(self._open) if o]

    @property
    def n_free_rows(self) -> int:
        return self._open.count(False)

    def open_row(self) -> int:
        """Take the lowest free row; its tables are empty, its state cleared."""
        for row, taken in enumerate(self._open):
            if not taken:
                break
        else:
            raise RuntimeError(f"all {self.max_rows} rows are open")
        self._open[row] = True
        self.scalars.clear(row)
        for s in self._slots:
            if isinstance(s, StateSlot):
                s.state[row].zero_()
        return row

    def close_row(self, row: int):
        """Give back everything the row holds."""
        self._check_open(row)
        for g in self.groups:
            g.release(row)
        self.scalars.clear(row)
        self._open[row] = False

    def move_row(self, src: int, dst: int):
        """Relocate an open row; only table rows and fixed-size state move, no page does
        (model/qwen/qwen_kv_paged.py:102-109)."""
        self._check_open(src)
        if self._open[dst]:
            raise ValueError(f"row {dst} is open; close it first")
        for g in self.groups:
            g.host_table[dst] = g.host_table[src]
            g.host_table[src] = NULL_PAGE
            g.covered[dst], g.covered[src] = g.covered[src], 0
            g.first_live[dst], g.first_live[src] = g.first_live[src], 0
            g.dirty.update((src, dst))
        for s in self._slots:
            if isinstance(s, StateSlot):
                s.state[dst].copy_(s.state[src])
        self.scalars.move(src, dst)
        self._open[dst], self._open[src] = True, False

    def _check_open(self, row: int):
        if not (0 <= row < self.max_rows) or not self._open[row]:
            raise ValueError(f"row {row} is not open")

    # -- pages -----------------------------------------------------------------------------
    def length(self, row: int) -> int:
        return int(self.scalars.length[row])

    def pages_short(self, row: int, new_len: int) -> int:
        """How many pages the fullest group lacks for ``row`` to grow to ``new_len``
        tokens, counting what the step itself would give back. 0 means it fits."""
        self._check_open(row)
        start = self.length(row)
        short = 0
        for g in self.groups:
            freed = g.droppable(row, start) - g.first_live[row]
            short = max(short, g.missing(row, new_len) - freed - g.allocator.n_free)
        return max(short, 0)

    def pages_needed(self, row: int, new_len: int):
        """Per group: pages ``row`` would take to grow to ``new_len`` tokens, minus the pages
        that step would give back first (may be negative)."""
        self._check_open(row)
        start = self.length(row)
        return [g.missing(row, new_len) - (g.droppable(row, start) - g.first_live[row])
                for g in self.groups]

    def free_pages(self):
        """Per group: pages free now."""
        return [g.allocator.n_free for g in self.groups]

    def held_pages(self, row: int):
        """Per group: pages ``row`` holds now."""
        return [g.covered[row] - g.first_live[row] for g in self.groups]

    @property
    def pool_tokens(self) -> int:
        """Tokens one request can hold if it has the whole pool of every group."""
        if not self.groups:
            return self.max_len
        return min(self.max_len, min(g.allocator.num_blocks for g in self.groups) * self.block_size)

    def reserve(self, row: int, new_len: int):
        """Make sure every group holds the pages for positions up to ``new_len`` of
        ``row``, after giving back the pages its next tokens can no longer see.
        Raises OutOfBlocks, with nothing taken, if any group cannot."""
        self._check_open(row)
        if new_len > self.max_len:
            raise ValueError(f"row {row}: {new_len} tokens exceed max_len {self.max_len}")
        start = self.length(row)
        for g in self.groups:
            g.drop_behind(row, start)
        for g in self.groups:
            if g.missing(row, new_len) > g.allocator.n_free:
                raise OutOfBlocks(f"row {row} needs {g.missing(row, new_len)} more pages to hold "
                                  f"{new_len} tokens, {g.allocator.n_free} free")
        for g in self.groups:
            g.extend(row, new_len)

    def advance(self, row: int, n_tokens: int):
        self.scalars.length[row] += n_tokens

    def sync(self):
        """Bring the device tables up to date with the host's."""
        for g in self.groups:
            g.sync()

    def slot(self, slot_id: int):
        return self._slots[slot_id]

    @property
    def null_row(self) -> int:
        """A row that is never opened: all its table entries are the null page."""
        return self.max_rows

    @property
    def n_free_pages(self) -> int:
        return min((g.allocator.n_free for g in self.groups), default=0)

    # -- invariants, for tests ---------------------------------------------------------------
    def check(self):
        """No page lost, held twice or held by a closed row; tables agree with the books."""
        for gi, g in enumerate(self.groups):
            seen = {}
            for row in range(self.max_rows):
                held = g.held_by(row)
                if not self._open[row] and (held or g.host_table[row].any()):
                    raise AssertionError(f"group {gi}: closed row {row} holds pages")
                outside = np.concatenate([g.host_table[row, :g.first_live[row]],
                                          g.host_table[row, g.covered[row]:]])
                if outside.any():
                    raise AssertionError(f"group {gi}: row {row} has table entries outside its live range")
                for p in held:
                    if p == NULL_PAGE:
                        raise AssertionError(f"group {gi}: row {row} holds the null page")
                    if p in seen:
                        raise AssertionError(f"group {gi}: page {p} held by rows {seen[p]} and {row}")
                    if not g.allocator.is_held(p):
                        raise AssertionError(f"group {gi}: page {p} in row {row} is marked free")
                    seen[p] = row
            if len(seen) + g.allocator.n_free != g.allocator.num_blocks:
                raise AssertionError(f"group {gi}: {len(seen)} held + {g.allocator.n_free} free != "
                                     f"{g.allocator.num_blocks}")
        return True
