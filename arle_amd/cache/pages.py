"""Page bookkeeping: a pool of page ids and per-request block tables for one group of layers.

Host-side only; nothing here touches the GPU, so all of it is tested on the CPU.
Behaviour follows the reference's pool (crates/cuda-kernels/src/paged_kv.rs):
LIFO free stack that hands out page 0 first (:416), tail page filled before a new
page is taken and all-or-nothing allocation (:498-533), pages returned when a
request ends (:985-1000).  Prefix sharing, reference counts and copy-on-write are
not part of this engine: a page has exactly one owner.

A group may have a window: keys older than `window` positions behind the newest
one are never read again, so the pages that hold only such keys are given back
while the request is still running (`trim`).
"""
from __future__ import annotations

from dataclasses import dataclass

FREED = -1  # block-table entry of a logical page that a window has passed


class OutOfPages(RuntimeError):
    """Not enough free pages; nothing was allocated."""


class PagePool:
    """Free stack over page ids 0..num_pages-1 with ownership checks."""

    def __init__(self, num_pages: int):
        if num_pages < 0:
            raise ValueError("num_pages must not be negative")
        self.num_pages = num_pages
        self._free = list(range(num_pages - 1, -1, -1))  # pop() yields 0 first
        self._held = [False] * num_pages

    @property
    def free_count(self) -> int:
        return len(self._free)

    def take(self, n: int) -> list:
        if n > len(self._free):
            raise OutOfPages(f"out of pages (requested {n} new pages, available {len(self._free)})")
        pages = [self._free.pop() for _ in range(n)]
        for p in pages:
            if self._held[p]:
                raise AssertionError(f"page {p} handed out twice")
            self._held[p] = True
        return pages

    def give_back(self, pages) -> None:
        for p in pages:
            if not 0 <= p < self.num_pages or not self._held[p]:
                raise AssertionError(f"page {p} freed twice or never held")
            self._held[p] = False
            self._free.append(p)

    def held_count(self) -> int:
        return sum(self._held)


@dataclass
class BlockTable:
    """Logical page -> physical page of one request in one group, and its length in tokens."""

    pages: list          # physical ids; FREED where a window has passed
    length: int = 0      # tokens written so far
    first_live: int = 0  # logical index of the first page still held


class PageGroup:
    """Pages and block tables of the layers that share one need (one page-id space)."""

    def __init__(self, num_pages: int, page_size: int, window: int | None = None):
        if page_size <= 0:
            raise ValueError("page_size must be positive")
        if window is not None and window <= 0:
            raise ValueError("window must be positive")
        self.page_size = page_size
        self.window = window
        self.pool = PagePool(num_pages)
        self.tables: dict = {}  # request key -> BlockTable

    # -- queries ------------------------------------------------------------------
    def pages_needed(self, key, n_tokens: int) -> int:
        """New pages that appending n tokens to `key` takes (tail room is used first)."""
        table = self.tables[key]
        have = len(table.pages) * self.page_size
        need = table.length + n_tokens
        return max(0, -(-(need - have) // self.page_size)) if need > have else 0

    def free_tokens(self) -> int:
        """Free pages in tokens plus the unused tail room of live requests (paged_kv.rs:1122-1137)."""
        tail = sum(len(t.pages) * self.page_size - t.length for t in self.tables.values())
        return self.pool.free_count * self.page_size + tail

    # -- changes ------------------------------------------------------------------
    def open(self, key) -> None:
        if key in self.tables:
            raise KeyError(f"request {key!r} already has a block table")
        self.tables[key] = BlockTable(pages=[])

    def append(self, key, n_tokens: int) -> list:
        """Make room for n more tokens; returns the (logical index, page) pairs newly mapped."""
        table = self.tables[key]
        new = self.pool.take(self.pages_needed(key, n_tokens))
        first = len(table.pages)
        table.pages.extend(new)
        table.length += n_tokens
        return [(first + i, p) for i, p in enumerate(new)]

    def truncate(self, key, new_length: int) -> list:
        """Drop tokens beyond new_length and whole trailing pages (paged_kv.rs:1004-1037)."""
        table = self.tables[key]
        if not 0 <= new_length <= table.length:
            raise ValueError("truncate: new length out of range")
        keep = -(-new_length // self.page_size)
        dropped = [(i, p) for i, p in enumerate(table.pages[keep:], start=keep)]
        self.pool.give_back([p for _, p in dropped if p != FREED])
        del table.pages[keep:]
        table.length = new_length
        table.first_live = min(table.first_live, keep)
        return dropped

    def trim(self, key) -> list:
        """Give back the pages every key of which the window has passed; returns their logical indices.

        After `length` tokens the next query sits at position >= length and reads keys
        > position - window, so key c is dead once c <= length - window.
        """
        if self.window is None:
            return []
        table = self.tables[key]
        dead_pages = max(0, (table.length - self.window + 1)) // self.page_size
        dead_pages = min(dead_pages, len(table.pages))
        freed = []
        for i in range(table.first_live, dead_pages):
            self.pool.give_back([table.pages[i]])
            table.pages[i] = FREED
            freed.append(i)
        table.first_live = max(table.first_live, dead_pages)
        return freed

    def close(self, key) -> None:
        table = self.tables.pop(key)
        self.pool.give_back([p for p in table.pages if p != FREED])

    # -- checks -------------------------------------------------------------------
    def check(self) -> None:
        """No page lost, held twice or freed twice."""
        owned = [p for t in self.tables.values() for p in t.pages if p != FREED]
        if len(owned) != len(set(owned)):
            raise AssertionError("a page is held by two requests")
        free = self.pool._free
        if len(free) != len(set(free)):
            raise AssertionError("a page is on the free stack twice")
        if set(owned) & set(free):
            raise AssertionError("a page is both held and free")
        if len(owned) + len(free) != self.pool.num_pages:
            raise AssertionError(
                f"pages lost: {len(owned)} held + {len(free)} free != {self.pool.num_pages}")
        if self.pool.held_count() != len(owned):
            raise AssertionError("held flags disagree with the block tables")
        for key, t in self.tables.items():
            if t.length > len(t.pages) * self.page_size:
                raise AssertionError(f"request {key!r} is longer than its pages")
