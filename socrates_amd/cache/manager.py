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

from ..parts.registry import PagedKV, PagedLatent, RowState
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
    # with pooled blocks (``PagedKV.pool``): the slot of the blocks' mean keys and values (its pages hold
    # ``block_size`` entries, entry b of a row stands for positions b * pool .. b * pool + pool - 1)
    pooled: Optional["PagedSlot"] = None
    pool: int = 0


@dataclass
class StateSlot:
    """What a mixer with fixed-size state sees: float32 [max_rows, *shape]."""
    state: torch.Tensor


class PagedGroup:
    """Cache slots with the same need: one allocator, one table, a pool pair per slot."""

    def __init__(self, need: PagedKV, max_rows, table_width, block_size, num_blocks, dtype, device, per=0):
        """``per``: positions that one entry of a page stands for (0: a token; P >= 1: the mean of a block of P
        tokens, which exists once the block is complete and is never given back before the row closes)."""
        self.need, self.block_size, self.table_width = need, block_size, table_width
        self.means, self.per = per > 0, max(per, 1)
        self.allocator = BlockAllocator(num_blocks)
        # one row more than can be opened: the null row, whose entries all point at the null
        # page, stands in for the padding rows of a fixed-width (captured) decode step
        self.host_table = np.zeros((max_rows + 1, table_width), dtype=np.int32)
        self.table = torch.zeros((max_rows + 1, table_width), dtype=torch.int32, device=device)
        # per row: number of logical blocks ever covered, and the first one still held
        self.covered = [0] * max_rows
        self.first_live = [0] * max_rows
        # with a window that keeps the first positions visible: the blocks that hold them stay with the
        # row whatever the window has passed (a row then holds blocks 0 .. kept and first_live .. covered)
        keep_first = getattr(need, "keep_first", 0) if need.window is not None and not self.means else 0
        self.kept_blocks = blocks_for(keep_first, block_size) if keep_first > 0 else 0
        self.dirty = set()
        # a latent is kept as one "head" of ``width`` elements, in one pool per slot
        self.pool_shape = ((num_blocks + 1, 1, block_size, need.width) if isinstance(need, PagedLatent)
                           else (num_blocks + 1, need.n_kv_heads, block_size, need.head_dim))
        self.dtype, self.device = dtype, device
        self.pools = {}
        self._upload = PinnedUploader(device) if torch.device(device).type == "cuda" else None

    def add_slot(self, slot_id: int):
        k = torch.zeros(self.pool_shape, dtype=self.dtype, device=self.device)
        # (a latent serves as keys and as values: both names point at the one pool)
        v = k if isinstance(self.need, PagedLatent) else torch.zeros(self.pool_shape, dtype=self.dtype, device=self.device)
        self.pools[slot_id] = (k, v)

    # -- pages a row needs / can drop ---------------------------------------------------------
    def droppable(self, row: int, next_start: int) -> int:
        """Logical blocks of ``row`` that no token at position >= next_start can see."""
        if self.need.window is None or self.means:
            return self.first_live[row]
        first_visible = max(0, next_start - self.need.window + 1)
        pool = getattr(self.need, "pool", 0)
        if pool:
            # the block that holds next_start is not complete: its tokens stay until its mean is taken
            first_visible = min(first_visible, next_start // pool * pool)
        return max(self.first_live[row], min(first_visible // self.block_size, self.covered[row]))

    def _held(self, row: int):
        """The logical blocks ``row`` holds: the kept first ones and those from first_live on."""
        a = min(self.kept_blocks, self.covered[row])
        b = max(self.first_live[row], a)
        return list(range(a)) + list(range(b, self.covered[row]))

    def would_free(self, row: int, next_start: int) -> int:
        """How many pages ``drop_behind`` would give back."""
        return max(0, self.droppable(row, next_start) - max(self.first_live[row], min(self.kept_blocks, self.covered[row])))

    def held_count(self, row: int) -> int:
        return len(self._held(row))

    def missing(self, row: int, new_len: int) -> int:
        return max(0, blocks_for(new_len // self.per, self.block_size) - self.covered[row])

    def drop_behind(self, row: int, next_start: int):
        upto = self.droppable(row, next_start)
        lo = max(self.first_live[row], min(self.kept_blocks, self.covered[row]))
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
                raise ValueError(f"{new_len} tokens need {lo + n} pages, the table holds {self.table_width}")
            self.host_table[row, lo:lo + n] = self.allocator.alloc(n)
            self.covered[row] = lo + n
            self.dirty.add(row)

    def release(self, row: int):
        hi = self.covered[row]
        held = self._held(row)
        if held:
            self.allocator.free([int(p) for p in self.host_table[row, held]])
        if hi:
            self.host_table[row, :hi] = NULL_PAGE
            self.dirty.add(row)
        self.covered[row] = self.first_live[row] = 0

    def held_by(self, row: int):
        return [int(p) for p in self.host_table[row, self._held(row)]]

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
        """needs: per cache slot a PagedKV, a PagedLatent, a RowState or None (see parts.cache_needs).
        num_blocks: usable pages of every paged group (the null page comes on top)."""
        if block_size < 1 or max_rows < 1 or max_len < 1:
            raise ValueError("block_size, max_rows and max_len must be positive")
        self.max_rows, self.max_len, self.block_size = max_rows, max_len, block_size
        self.dtype, self.device = dtype, device
        self.table_width = blocks_for(max_len, block_size)
        self.groups: List[PagedGroup] = []
        self._slots = []
        self._by_need = {}
        self._num_blocks = num_blocks
        for slot_id, need in enumerate(needs):
            try:
                self._slots.append(self._make_slot(need))
            except (TypeError, ValueError) as e:
                raise type(e)(f"cache slot {slot_id}: {e}") from None
        self.scalars = RowScalars(max_rows)
        self._open = [False] * max_rows

    def _group(self, key, need, num_blocks, per=0):
        group = self._by_need.get(key)
        if group is None:
            table_width = self.table_width if not per else blocks_for(self.max_len // per, self.block_size)
            group = PagedGroup(need, self.max_rows, max(table_width, 1), self.block_size, num_blocks, self.dtype,
                               self.device, per=per)
            self._by_need[key] = group
            self.groups.append(group)
        return group

    def _make_slot(self, need):
        if isinstance(need, tuple):
            # a mixer made of several mixers: one slot for each, in order
            return tuple(self._make_slot(n) for n in need)
        if isinstance(need, (PagedKV, PagedLatent)):
            if getattr(need, "keep_first", 0) < 0:
                raise ValueError("keep_first is not negative")
            pool = getattr(need, "pool", 0)
            if pool < 0 or (pool and (need.window is None or need.keep_first)):
                raise ValueError("pooled blocks need a window, and no kept first positions")
            group = self._group(need, need, self._num_blocks)
            serial = len(group.pools)
            group.add_slot(serial)
            k, v = group.pools[serial]
            slot = PagedSlot(k, v, group.table, self.block_size, need.window)
            if pool:
                # the means of the blocks stay with a row however far its window has moved on, so every row can
                # hold those of max_len tokens (a pool-th of what the tokens themselves would take)
                per_row = max(1, blocks_for(self.max_len // pool, self.block_size))
                means = self._group(("means", need), need, self.max_rows * per_row, per=pool)
                means.add_slot(serial)
                mk, mv = means.pools[serial]
                slot.pooled, slot.pool = PagedSlot(mk, mv, means.table, self.block_size, None), pool
            return slot
        if isinstance(need, RowState):
            kinds = {"float32": torch.float32, "int32": torch.int32, "compute": self.dtype}
            if need.dtype not in kinds:
                raise ValueError(f"a row's state is one of {sorted(kinds)}, not {need.dtype!r}")
            state = torch.zeros((self.max_rows + 1,) + tuple(need.shape), dtype=kinds[need.dtype], device=self.device)
            return StateSlot(state)
        if need is None:
            return None
        raise TypeError(f"unknown kind of need {need!r}")

    def _state_slots(self):
        def walk(slots):
            for s in slots:
                if isinstance(s, tuple):
                    yield from walk(s)
                elif isinstance(s, StateSlot):
                    yield s
        return walk(self._slots)

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
        for s in self._state_slots():
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
        for s in self._state_slots():
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
            short = max(short, g.missing(row, new_len) - g.would_free(row, start) - g.allocator.n_free)
        return max(short, 0)

    def pages_needed(self, row: int, new_len: int):
        """Per group: pages ``row`` would take to grow to ``new_len`` tokens, minus the pages
        that step would give back first (may be negative)."""
        self._check_open(row)
        start = self.length(row)
        return [g.missing(row, new_len) - g.would_free(row, start) for g in self.groups]

    def free_pages(self):
        """Per group: pages free now."""
        return [g.allocator.n_free for g in self.groups]

    def held_pages(self, row: int):
        """Per group: pages ``row`` holds now."""
        return [g.held_count(row) for g in self.groups]

    @property
    def pool_tokens(self) -> int:
        """Tokens one request can hold if it has the whole pool of every group."""
        if not self.groups:
            return self.max_len
        return min(self.max_len, min(g.allocator.num_blocks * g.per for g in self.groups) * self.block_size)

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
                live = np.zeros(g.table_width, dtype=bool)
                live[g._held(row)] = True
                if g.host_table[row, ~live].any():
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
