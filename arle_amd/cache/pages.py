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

import ctypes
from collections.abc import Mapping
from dataclasses import dataclass

from . import native

FREED = -1  # block-table entry of a logical page that a window has passed


class OutOfPages(RuntimeError):
    """Not enough free pages; nothing was allocated."""


class PagePool:
    """Free stack over page ids 0..num_pages-1 with ownership checks (a view of the native group's pool)."""

    def __init__(self, num_pages: int, _handle=None):
        if num_pages < 0:
            raise ValueError("num_pages must not be negative")
        self.num_pages = num_pages
        self._lib = native.lib()
        self._own = _handle is None
        self._h = _handle if _handle is not None else self._lib.arle_group_create(num_pages, 1, 0)

    def __del__(self):
        if getattr(self, "_own", False) and getattr(self, "_h", None):
            self._lib.arle_group_destroy(self._h)
            self._h = None

    @property
    def free_count(self) -> int:
        return self._lib.arle_group_free_count(self._h)

    def take(self, n: int) -> list:
        out = native.int_array(n)
        if self._lib.arle_group_take(self._h, n, out) < 0:
            raise OutOfPages(f"out of pages (requested {n} new pages, available {self.free_count})")
        return list(out[:n])

    def give_back(self, pages) -> None:
        pages = list(pages)
        arr = (ctypes.c_int * max(len(pages), 1))(*pages)
        if self._lib.arle_group_give_back(self._h, arr, len(pages)) < 0:
            raise AssertionError("a page was freed twice or never held")

    def held_count(self) -> int:
        return self._lib.arle_group_held_count(self._h)


@dataclass
class BlockTable:
    """Logical page -> physical page of one request in one group, and its length in tokens (a snapshot)."""

    pages: list          # physical ids; FREED where a window has passed
    length: int = 0      # tokens written so far
    first_live: int = 0  # logical index of the first page still held


class _Tables(Mapping):
    """request key -> BlockTable snapshot, read from the native group."""

    def __init__(self, group):
        self._g = group

    def __getitem__(self, key) -> BlockTable:
        return self._g._snapshot(key)

    def __iter__(self):
        return iter(self._g._ids)

    def __len__(self) -> int:
        return len(self._g._ids)

    def __contains__(self, key) -> bool:
        return key in self._g._ids


class PageGroup:
    """Pages and block tables of the layers that share one need (one page-id space).

    The bookkeeping lives in the native runtime core; request keys (any hashable) are mapped to
    integers here."""

    def __init__(self, num_pages: int, page_size: int, window: int | None = None):
        if page_size <= 0:
            raise ValueError("page_size must be positive")
        if window is not None and window <= 0:
            raise ValueError("window must be positive")
        if num_pages < 0:
            raise ValueError("num_pages must not be negative")
        self.page_size = page_size
        self.window = window
        self._lib = native.lib()
        self._h = self._lib.arle_group_create(num_pages, page_size, window or 0)
        self.pool = PagePool(num_pages, _handle=self._h)
        self._ids: dict = {}     # request key -> native id
        self._next_id = 0
        self.tables = _Tables(self)

    def __del__(self):
        if getattr(self, "_h", None):
            self._lib.arle_group_destroy(self._h)
            self._h = None

    def _id(self, key) -> int:
        return self._ids[key]          # KeyError for a request without a block table

    def _snapshot(self, key) -> BlockTable:
        kid = self._id(key)
        length, first = ctypes.c_int(), ctypes.c_int()
        n = self._lib.arle_group_table(self._h, kid, native.int_array(0), 0, ctypes.byref(length), ctypes.byref(first))
        buf = native.int_array(n)
        self._lib.arle_group_table(self._h, kid, buf, n, ctypes.byref(length), ctypes.byref(first))
        return BlockTable(pages=list(buf[:n]), length=length.value, first_live=first.value)

    # -- queries ------------------------------------------------------------------
    def pages_needed(self, key, n_tokens: int) -> int:
        """New pages that appending n tokens to `key` takes (tail room is used first)."""
        return self._lib.arle_group_pages_needed(self._h, self._id(key), n_tokens)

    def free_tokens(self) -> int:
        """Free pages in tokens plus the unused tail room of live requests (paged_kv.rs:1122-1137)."""
        return self._lib.arle_group_free_tokens(self._h)

    # -- changes ------------------------------------------------------------------
    def open(self, key) -> None:
        if key in self._ids:
            raise KeyError(f"request {key!r} already has a block table")
        self._ids[key] = self._next_id
        self._next_id += 1
        self._lib.arle_group_open(self._h, self._ids[key])

    def append(self, key, n_tokens: int) -> list:
        """Make room for n more tokens; returns the (logical index, page) pairs newly mapped."""
        kid = self._id(key)
        cap = self._lib.arle_group_pages_needed(self._h, kid, n_tokens)
        first, buf = ctypes.c_int(), native.int_array(cap)
        n = self._lib.arle_group_append(self._h, kid, n_tokens, ctypes.byref(first), buf, cap)
        if n == native.OUT_OF_PAGES:
            raise OutOfPages(f"out of pages (requested {cap} new pages, available {self.pool.free_count})")
        if n < 0:
            raise AssertionError(f"append failed with code {n}")
        return [(first.value + i, buf[i]) for i in range(n)]

    def truncate(self, key, new_length: int) -> list:
        """Drop tokens beyond new_length and whole trailing pages (paged_kv.rs:1004-1037)."""
        kid = self._id(key)
        cap = len(self._snapshot(key).pages)
        logical, pages = native.int_array(cap), native.int_array(cap)
        n = self._lib.arle_group_truncate(self._h, kid, new_length, logical, pages, cap)
        if n == native.OUT_OF_RANGE:
            raise ValueError("truncate: new length out of range")
        if n < 0:
            raise AssertionError(f"truncate failed with code {n}")
        return [(logical[i], pages[i]) for i in range(n)]

    def trim(self, key) -> list:
        """Give back the pages every key of which the window has passed; returns their logical indices."""
        if self.window is None:
            return []
        kid = self._id(key)
        cap = len(self._snapshot(key).pages)
        logical = native.int_array(cap)
        n = self._lib.arle_group_trim(self._h, kid, logical, cap)
        if n < 0:
            raise AssertionError(f"trim failed with code {n}")
        return list(logical[:n])

    def close(self, key) -> None:
        kid = self._ids.pop(key)
        if self._lib.arle_group_close(self._h, kid) < 0:
            raise AssertionError("close: a page was freed twice or never held")

    # -- checks -------------------------------------------------------------------
    def check(self) -> None:
        """No page lost, held twice or freed twice."""
        msg = ctypes.create_string_buffer(256)
        if self._lib.arle_group_check(self._h, msg, 256):
            raise AssertionError(msg.value.decode())
