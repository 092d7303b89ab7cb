"""The cache manager: paged keys/values per group of layers, and fixed-size state slots.

Every schedule entry of a model that owns a cache declares its need:
`PagedNeed` (keys and values per token: attention, possibly windowed) or `StateNeed`
(a block of fixed size per request: recurrent or convolutional state).  Entries with
equal paged needs form a group with one page-id space, one block table per request
and one pair of buffers `[entries, pages, kv_heads, page_size, head_dim]`.  State needs
get `[slots, *shape]` buffers, zeroed when a slot is assigned.  A request holds one
slot for its life; the slot is its row in every block table and state buffer.

The bookkeeping is host-side and works without a GPU (`device=None`), which is how the
CPU tests drive it.  Reference: one pool, one table per slot, per-slot model state
(crates/cuda-kernels/src/paged_kv.rs:34-102; infer/src/scheduler/cuda/core/construction.rs:119-203).
"""
from __future__ import annotations

from dataclasses import dataclass

import numpy as np
import torch

from .pages import FREED, OutOfPages, PageGroup


@dataclass(frozen=True)
class PagedNeed:
    num_kv_heads: int
    head_dim: int
    window: int | None = None  # None: every earlier key is kept


@dataclass(frozen=True)
class StateNeed:
    shape: tuple
    dtype: torch.dtype = torch.float32


@dataclass
class PagedView:
    """What a mixer sees of its paged cache during a step."""

    k_pages: torch.Tensor | None   # [pages, kv_heads, page_size, head_dim]
    v_pages: torch.Tensor | None   # [pages, kv_heads, head_dim, page_size]  (d-major inside a page)
    block_table: torch.Tensor | None  # int32 [slots, max_pages_per_request], shared by the group
    page_size: int
    window: int | None
    writes: bool                   # False for an entry that reads another entry's cache


@dataclass
class StateView:
    state: torch.Tensor | None     # [slots, *shape]


class NoFreeSlot(RuntimeError):
    pass


class CacheManager:
    def __init__(self, needs, *, page_size: int, num_pages: int, max_slots: int,
                 max_request_tokens: int, device=None, dtype: torch.dtype = torch.float32,
                 readers: dict | None = None):
        """
        needs: one entry per schedule entry: PagedNeed, StateNeed or None.
        readers: {entry index -> entry index whose cache it reads} for entries that own none.
        num_pages: pages of every paged group (each group has its own ids and buffers).
        max_request_tokens: longest request; fixes the width of the block tables.
        """
        self.page_size = page_size
        self.max_slots = max_slots
        self.device = device
        self.dtype = dtype
        self.max_pages_per_request = max(1, -(-max_request_tokens // page_size))
        self.needs = list(needs)
        self.readers = dict(readers or {})

        self.groups: list = []          # PageGroup
        self._group_needs: list = []    # PagedNeed of each group
        self._group_entries: list = []  # schedule entries of each group, in order
        self._entry_place: dict = {}    # entry -> (group index, index within group)
        for entry, need in enumerate(self.needs):
            if isinstance(need, PagedNeed):
                if need not in self._group_needs:
                    self._group_needs.append(need)
                    self._group_entries.append([])
                    self.groups.append(PageGroup(num_pages, page_size, need.window))
                g = self._group_needs.index(need)
                self._entry_place[entry] = (g, len(self._group_entries[g]))
                self._group_entries[g].append(entry)

        # slots
        self._free_slots = list(range(max_slots - 1, -1, -1))
        self.slot_of: dict = {}         # request key -> slot
        self._lengths: dict = {}        # request key -> tokens appended so far

        # host mirrors of the block tables, one per group
        self._tables_host = [np.full((max_slots, self.max_pages_per_request), 0, dtype=np.int32)
                             for _ in self.groups]
        self._dirty = [set() for _ in self.groups]

        # device buffers
        self.k_buffers, self.v_buffers, self.tables_dev, self.state_buffers = [], [], [], {}
        if device is not None:
            for g, need in enumerate(self._group_needs):
                n = len(self._group_entries[g])
                # keys [.., slot in page, d]; values d-major inside a page [.., d, slot in page]
                self.k_buffers.append(torch.zeros((n, num_pages, need.num_kv_heads, page_size, need.head_dim),
                                                  dtype=dtype, device=device))
                self.v_buffers.append(torch.zeros((n, num_pages, need.num_kv_heads, need.head_dim, page_size),
                                                  dtype=dtype, device=device))
                self.tables_dev.append(torch.zeros((max_slots, self.max_pages_per_request),
                                                   dtype=torch.int32, device=device))
            for entry, need in enumerate(self.needs):
                if isinstance(need, StateNeed):
                    self.state_buffers[entry] = torch.zeros((max_slots, *need.shape),
                                                            dtype=need.dtype, device=device)

    # -- requests -------------------------------------------------------------------
    def admit(self, key) -> int:
        """Give a request a slot and empty block tables; its state blocks are zeroed."""
        if key in self.slot_of:
            raise KeyError(f"request {key!r} is already live")
        if not self._free_slots:
            raise NoFreeSlot(f"all {self.max_slots} slots are taken")
        slot = self._free_slots.pop()
        self.slot_of[key] = slot
        self._lengths[key] = 0
        for group in self.groups:
            group.open(key)
        for buf in self.state_buffers.values():
            buf[slot].zero_()
        return slot

    def release(self, key) -> None:
        """End of a request: every page it holds and its slot go back."""
        slot = self.slot_of.pop(key)
        del self._lengths[key]
        for group in self.groups:
            group.close(key)
        self._free_slots.append(slot)

    def is_live(self, key) -> bool:
        return key in self.slot_of

    def length(self, key) -> int:
        """Tokens of the request that the cache holds (written by completed appends)."""
        return self._lengths[key]

    @property
    def free_slot_count(self) -> int:
        return len(self._free_slots)

    # -- pages ----------------------------------------------------------------------
    def pages_needed(self, appends) -> list:
        """Per group, the new pages that `appends` = [(key, n_tokens)] take together."""
        return [sum(group.pages_needed(k, n) for k, n in appends) for group in self.groups]

    def can_append(self, appends) -> bool:
        return all(need <= group.pool.free_count
                   for need, group in zip(self.pages_needed(appends), self.groups))

    def free_pages(self) -> list:
        return [g.pool.free_count for g in self.groups]

    def free_tokens(self) -> int:
        return min((g.free_tokens() for g in self.groups), default=0)

    def append(self, appends) -> None:
        """Room for n more tokens of each request, in every group; all or nothing."""
        for key, n in appends:
            if key not in self.slot_of:
                raise KeyError(f"request {key!r} is not live")
            if n <= 0:
                raise ValueError("append: token count must be positive")
            if self.groups and self.length(key) + n > self.max_pages_per_request * self.page_size:
                raise OutOfPages(f"request {key!r} would exceed the longest request the block "
                                 f"tables were sized for ({self.max_pages_per_request * self.page_size} tokens)")
        needs = self.pages_needed(appends)
        for g, (need, group) in enumerate(zip(needs, self.groups)):
            if need > group.pool.free_count:
                raise OutOfPages(f"group {g}: out of pages (requested {need} new pages for "
                                 f"{sum(n for _, n in appends)} tokens, available {group.pool.free_count})")
        for g, group in enumerate(self.groups):
            for key, n in appends:
                slot = self.slot_of[key]
                for logical, page in group.append(key, n):
                    self._tables_host[g][slot, logical] = page
                    self._dirty[g].add(slot)
        for key, n in appends:
            self._lengths[key] += n

    def truncate(self, key, new_length: int) -> None:
        if not 0 <= new_length <= self._lengths[key]:
            raise ValueError("truncate: new length out of range")
        for group in self.groups:
            group.truncate(key, new_length)
        self._lengths[key] = new_length

    def trim_windows(self, key) -> None:
        """Give back pages that a window has passed (after a step is complete)."""
        for group in self.groups:
            group.trim(key)

    # -- views for the step -----------------------------------------------------------
    def sync_tables(self) -> None:
        """Copy block-table rows that changed since the last call to the GPU."""
        if self.device is None:
            return
        for g in range(len(self.groups)):
            if not self._dirty[g]:
                continue
            rows = sorted(self._dirty[g])
            host = torch.from_numpy(self._tables_host[g][rows])
            self.tables_dev[g][torch.tensor(rows, device=self.device)] = host.to(self.device)
            self._dirty[g].clear()

    def view(self, entry: int):
        """The cache of a schedule entry: its own, or the one it was told to read."""
        owner = self.readers.get(entry, entry)
        need = self.needs[owner] if owner < len(self.needs) else None
        if isinstance(need, PagedNeed):
            g, idx = self._entry_place[owner]
            has = self.device is not None
            return PagedView(k_pages=self.k_buffers[g][idx] if has else None,
                             v_pages=self.v_buffers[g][idx] if has else None,
                             block_table=self.tables_dev[g] if has else None,
                             page_size=self.page_size, window=need.window, writes=owner == entry)
        if isinstance(need, StateNeed):
            return StateView(state=self.state_buffers.get(owner))
        return None

    def table_of(self, key, group: int = 0) -> list:
        return list(self.groups[group].tables[key].pages)

    # -- checks -----------------------------------------------------------------------
    def check(self) -> None:
        for group in self.groups:
            group.check()
            if set(group.tables) != set(self.slot_of):
                raise AssertionError("block tables and slots name different requests")
        slots = list(self.slot_of.values())
        if len(slots) != len(set(slots)) or set(slots) & set(self._free_slots):
            raise AssertionError("a slot is held twice or both held and free")
        if len(slots) + len(self._free_slots) != self.max_slots:
            raise AssertionError("slots lost")
        for k in self.slot_of:
            for g in self.groups:
                if g.tables[k].length != self._lengths[k]:
                    raise AssertionError(f"a group disagrees on the length of {k!r}")


__all__ = ["CacheManager", "PagedNeed", "StateNeed", "PagedView", "StateView", "OutOfPages",
           "NoFreeSlot", "FREED"]
