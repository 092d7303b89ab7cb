"""The cache manager: paged keys/values per group of layers, and fixed-size state slots.

Every schedule entry of a model that owns a cache declares its need:
`PagedNeed` (tensors that grow by one slot per token: attention, possibly windowed) or
`StateNeed` (a block of fixed size per request: recurrent or convolutional state).  A paged
need lists its own tensors (`PageTensor`: a name, the shape of one page with the token axis
marked, an element type): keys and values `[kv_heads, page, head_dim]` / `[kv_heads, head_dim,
page]` unless it says otherwise, so a mixer that caches one compressed vector per token, or
keeps its cache in another type than the activations, declares that and nothing here
changes.  Entries with equal paged needs form a group with one page-id space, one block
table per request and one buffer `[entries, pages, *page shape]` per declared tensor.  State
needs get `[slots, *shape]` buffers, zeroed when a slot is assigned.  A request holds one
slot for its life; the slot is its row in every block table and state buffer.

The bookkeeping is host-side and works without a GPU (`device=None`), which is how the
CPU tests drive it.  Reference: one pool, one table per slot, per-slot model state
(crates/cuda-kernels/src/paged_kv.rs:34-102; infer/src/scheduler/cuda/core/construction.rs:119-203).
"""
from __future__ import annotations

from dataclasses import dataclass

import numpy as np
import torch

from ..kernels.upload import upload
from .pages import FREED, OutOfPages, PageGroup


PAGE = "page"   # stands for the token axis (length page_size) in the shape of a PageTensor


@dataclass(frozen=True)
class PageTensor:
    """One tensor of a paged need: `shape` is that of one page, with PAGE where the tokens of the page go."""

    name: str
    shape: tuple
    dtype: torch.dtype | None = None   # None: the engine's activation type

    def page_shape(self, page_size: int) -> tuple:
        if sum(1 for d in self.shape if d == PAGE) != 1:
            raise ValueError(f"page tensor {self.name!r}: the shape must hold the token axis PAGE exactly once")
        return tuple(page_size if d == PAGE else int(d) for d in self.shape)

    def bytes_per_token(self, act_dtype: torch.dtype) -> int:
        n = 1
        for d in self.page_shape(1):
            n *= d
        return n * torch.empty((), dtype=self.dtype or act_dtype).element_size()


@dataclass(frozen=True)
class PagedNeed:
    """Keys and values of num_kv_heads x head_dim per token, or the `tensors` the mixer lists itself."""

    num_kv_heads: int = 0
    head_dim: int = 0
    window: int | None = None  # None: every earlier token is kept
    tensors: tuple = ()        # of PageTensor; empty: "k" [kv_heads, PAGE, head_dim] and "v" [kv_heads, head_dim, PAGE]
    page_size: int | None = None   # tokens a page of this need holds; None: the manager's own page length

    def page_tensors(self) -> tuple:
        if self.tensors:
            names = [t.name for t in self.tensors]
            if len(set(names)) != len(names):
                raise ValueError(f"a paged need names a tensor twice: {names}")
            return tuple(self.tensors)
        if self.num_kv_heads <= 0 or self.head_dim <= 0:
            raise ValueError("a paged need gives num_kv_heads and head_dim, or its own tensors")
        # keys [.., slot in page, d]; values d-major inside a page [.., d, slot in page]
        return (PageTensor("k", (self.num_kv_heads, PAGE, self.head_dim)),
                PageTensor("v", (self.num_kv_heads, self.head_dim, PAGE)))

    def bytes_per_token(self, act_dtype: torch.dtype) -> int:
        return sum(t.bytes_per_token(act_dtype) for t in self.page_tensors())


@dataclass(frozen=True)
class StateNeed:
    shape: tuple
    dtype: torch.dtype = torch.float32

    def bytes_per_slot(self) -> int:
        n = 1
        for d in self.shape:
            n *= int(d)
        return n * torch.empty((), dtype=self.dtype).element_size()


def cache_bytes_per_token(needs, act_dtype: torch.dtype) -> int:
    """Bytes one token takes over every schedule entry that owns a paged cache.  For keys and values of every
    layer this is the reference's 2 * layers * kv_heads * head_dim * element size
    (infer/src/model/qwen3/forward.rs:777-783)."""
    return sum(n.bytes_per_token(act_dtype) for n in needs if isinstance(n, PagedNeed))


def state_bytes_per_slot(needs) -> int:
    return sum(n.bytes_per_slot() for n in needs if isinstance(n, StateNeed))


def pages_for_memory(free_bytes: int, total_bytes: int, mem_fraction_static: float, bytes_per_page: int,
                     reserved_bytes: int = 0, most_pages: int | None = None) -> int:
    """Pages of a pool sized from the GPU's memory, as the reference sizes its pool
    (infer/src/scheduler/cuda/core/construction.rs:131-203): what is free now (the weights are loaded), less a
    headroom of (1 - mem_fraction_static) of the whole memory for activations and workspaces, less what else is
    reserved (state slots), divided by a page's bytes over all layers.  `most_pages`: what all slots can hold at
    their longest; more would never be used, since pages are not shared between requests."""
    if not 0.0 < mem_fraction_static <= 1.0:
        raise ValueError("mem_fraction_static must be in (0, 1]")     # infer/src/scheduler/types.rs:407-409
    if bytes_per_page <= 0:
        return 0
    headroom = int(total_bytes * (1.0 - mem_fraction_static))
    budget = max(0, int(free_bytes) - headroom - int(reserved_bytes))
    pages = budget // bytes_per_page
    return int(min(pages, most_pages) if most_pages is not None else pages)


AUTO_SLOTS_MIN, AUTO_SLOTS_MAX = 4, 128       # infer/src/main.rs:807-808


def slots_for_tokens(cache_tokens: int, longest_request: int) -> int:
    """How many requests run at a time when the caller does not say: as many of the longest length as the cache
    holds, no fewer than 4 and no more than 128 (the reference's server: infer/src/main.rs:782-855)."""
    return max(AUTO_SLOTS_MIN, min(AUTO_SLOTS_MAX, int(cache_tokens) // max(1, int(longest_request))))


@dataclass
class PagedView:
    """What a mixer sees of its paged cache during a step."""

    pages: dict                    # tensor name -> [pages, *page shape]  (None values without a device)
    block_table: torch.Tensor | None  # int32 [slots, max_pages_per_request], shared by the group
    page_size: int
    window: int | None
    writes: bool                   # False for an entry that reads another entry's cache

    @property
    def k_pages(self):             # [pages, kv_heads, page_size, head_dim]
        return self.pages["k"]

    @property
    def v_pages(self):             # [pages, kv_heads, head_dim, page_size]  (d-major inside a page)
        return self.pages["v"]


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
        page_size, num_pages: page length and pages of every paged group (each group has its own ids and
            buffers).  A need that names a page length of its own gets pages of that length, as many as hold
            the same number of tokens (num_pages * page_size), and block tables of its own width.
        max_request_tokens: longest request; fixes the width of the block tables.
        """
        self.page_size = page_size
        self.max_slots = max_slots
        self.device = device
        self.dtype = dtype
        self.max_pages_per_request = max(1, -(-max_request_tokens // page_size))   # of a group with the default page length
        self.needs = list(needs)
        self.readers = dict(readers or {})

        self.groups: list = []          # PageGroup
        self._group_needs: list = []    # PagedNeed of each group
        self._group_entries: list = []  # schedule entries of each group, in order
        self._entry_place: dict = {}    # entry -> (group index, index within group)
        for entry, need in enumerate(self.needs):
            if isinstance(need, PagedNeed):
                if need not in self._group_needs:
                    own = int(need.page_size or page_size)
                    if own <= 0:
                        raise ValueError("a paged need's page_size must be positive")
                    self._group_needs.append(need)
                    self._group_entries.append([])
                    self.groups.append(PageGroup(num_pages if own == page_size else (num_pages * page_size) // own,
                                                 own, need.window))
                g = self._group_needs.index(need)
                self._entry_place[entry] = (g, len(self._group_entries[g]))
                self._group_entries[g].append(entry)

        # slots
        self._free_slots = list(range(max_slots - 1, -1, -1))
        self.slot_of: dict = {}         # request key -> slot
        self._lengths: dict = {}        # request key -> tokens appended so far

        # the longest request that every group's block table can map
        self._table_widths = [max(1, -(-max_request_tokens // g.page_size)) for g in self.groups]
        self.request_capacity = min((w * g.page_size for w, g in zip(self._table_widths, self.groups)),
                                    default=self.max_pages_per_request * page_size)
        # host mirrors of the block tables, one per group
        self._tables_host = [np.full((max_slots, w), 0, dtype=np.int32) for w in self._table_widths]
        self._dirty = [set() for _ in self.groups]

        # device buffers
        self.page_buffers, self.tables_dev, self.state_buffers = [], [], {}   # page_buffers[g]: name -> tensor
        for need in self._group_needs:
            need.page_tensors()     # a need that is not well formed fails here, with or without a device
        if device is not None:
            for g, need in enumerate(self._group_needs):
                n = len(self._group_entries[g])
                group = self.groups[g]
                self.page_buffers.append({
                    t.name: torch.zeros((n, group.pool.num_pages, *t.page_shape(group.page_size)),
                                        dtype=t.dtype or dtype, device=device)
                    for t in need.page_tensors()})
                self.tables_dev.append(torch.zeros((max_slots, self._table_widths[g]), dtype=torch.int32, device=device))
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

    def pool_tokens(self) -> int:
        """Tokens that the smallest group's pages hold in all."""
        return min((g.pool.num_pages * g.page_size for g in self.groups), default=1 << 30)

    def pages_for_length(self, tokens: int) -> list:
        """Per group, the pages that a request of `tokens` tokens maps (before any window gives some back)."""
        return [-(-int(tokens) // g.page_size) for g in self.groups]

    def append(self, appends) -> None:
        """Room for n more tokens of each request, in every group; all or nothing."""
        for key, n in appends:
            if key not in self.slot_of:
                raise KeyError(f"request {key!r} is not live")
            if n <= 0:
                raise ValueError("append: token count must be positive")
            if self.groups and self.length(key) + n > self.request_capacity:
                raise OutOfPages(f"request {key!r} would exceed the longest request the block "
                                 f"tables were sized for ({self.request_capacity} tokens)")
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

    # -- state slots across a step that may fail ----------------------------------------
    def snapshot_state(self, keys):
        """A copy of the state blocks of these requests, to be handed to `restore_state` if the step that is
        about to overwrite them fails; None when no entry keeps state.  [requests of the step, *shape] each."""
        if not self.state_buffers:
            return None
        rows = torch.tensor([self.slot_of[k] for k in keys], dtype=torch.long, device=self.device)
        return rows, {entry: buf.index_select(0, rows) for entry, buf in self.state_buffers.items()}

    def restore_state(self, snapshot) -> None:
        if snapshot is None:
            return
        rows, saved = snapshot
        for entry, values in saved.items():
            self.state_buffers[entry].index_copy_(0, rows, values)

    # -- views for the step -----------------------------------------------------------
    def sync_tables(self) -> None:
        """Copy block-table rows that changed since the last call to the GPU."""
        if self.device is None:
            return
        for g in range(len(self.groups)):
            if not self._dirty[g]:
                continue
            rows = sorted(self._dirty[g])
            # row numbers and rows in one staged copy that the host does not wait for
            staged = np.concatenate([np.asarray(rows, dtype=np.int32),
                                     self._tables_host[g][rows].astype(np.int32, copy=False).reshape(-1)])
            both = upload(staged, self.device)
            self.tables_dev[g].index_copy_(0, both[:len(rows)].long(), both[len(rows):].view(len(rows), -1))
            self._dirty[g].clear()

    def view(self, entry: int):
        """The cache of a schedule entry: its own, or the one it was told to read."""
        owner = self.readers.get(entry, entry)
        need = self.needs[owner] if owner < len(self.needs) else None
        if isinstance(need, PagedNeed):
            g, idx = self._entry_place[owner]
            has = self.device is not None
            pages = {t.name: (self.page_buffers[g][t.name][idx] if has else None) for t in need.page_tensors()}
            return PagedView(pages=pages, block_table=self.tables_dev[g] if has else None,
                             page_size=self.groups[g].page_size, window=need.window, writes=owner == entry)
        if isinstance(need, StateNeed):
            return StateView(state=self.state_buffers.get(owner))
        return None

    def bytes_per_token(self) -> int:
        return cache_bytes_per_token(self.needs, self.dtype)

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


__all__ = ["CacheManager", "PagedNeed", "PageTensor", "PAGE", "StateNeed", "PagedView", "StateView", "OutOfPages",
           "NoFreeSlot", "FREED", "cache_bytes_per_token", "state_bytes_per_slot", "pages_for_memory"]
