"""Host-side ownership of one group's physical pages.

Reference behaviour followed (flow_engine/cache.py:24-91): a reference count per
page, a LIFO free list, `allocate` evicting least-recently-used prefix entries
when the free list is short, `release` with an underflow check, and a prefix
index keyed by chained SHA-256 over (namespace, parent key, the block's tokens
as little-endian int64); only full blocks are keyed, lookup never covers the
last prompt token, a page is free only when neither a request nor the index
holds it.

Added: `promised` pages. A request may be promised pages at admission that it
takes later, one by one; promised pages cannot be given to anyone else.
"""
from __future__ import annotations

from collections import OrderedDict
import hashlib
import struct


class CapacityError(RuntimeError):
    """Not enough free pages (or state slots); the caller waits or refuses."""


class PagePool:
    def __init__(self, pages, page_size, prefix_cache=True):
        if pages <= 0 or page_size <= 0:
            raise ValueError("pages and page_size must be positive")
        self.capacity = int(pages)
        self.page_size = int(page_size)
        self.refs = [0] * self.capacity
        self.free = list(reversed(range(self.capacity)))
        self.prefixes: OrderedDict[bytes, int] = OrderedDict()
        self.prefix_cache = bool(prefix_cache)
        self.promised = 0
        self.hits = 0
        self.evictions = 0

    # ---- ownership ----------------------------------------------------
    def _release_one(self, page):
        if not 0 <= page < self.capacity:
            raise RuntimeError(f"page id {page} out of range")
        if self.refs[page] <= 0:
            raise RuntimeError("KV reference underflow")
        self.refs[page] -= 1
        if not self.refs[page]:
            self.free.append(page)

    def release(self, pages):
        for page in pages:
            if page >= 0:
                self._release_one(page)

    def _evictable(self):
        return sum(1 for page in self.prefixes.values() if self.refs[page] == 1)

    def available(self):
        """Pages that a new promise or an unpromised allocation could still get."""
        return len(self.free) + self._evictable() - self.promised

    def _make_room(self, count, others):
        # Evict least-recently-used prefix entries while the free list is short
        # (flow_engine/cache.py:49-54). An evicted entry whose page a request
        # still holds frees nothing; the loop goes on to the next entry.
        while len(self.free) - others < count and self.prefixes:
            _, page = self.prefixes.popitem(last=False)
            self._release_one(page)
            self.evictions += 1
        if len(self.free) - others < count:
            raise CapacityError("KV capacity exhausted; request must wait or reduce its token budget")

    def allocate(self, count, promised=0):
        """Take COUNT pages; PROMISED of them were promised to the caller before."""
        if count < 0 or promised < 0 or promised > count or promised > self.promised:
            raise ValueError("negative allocation")
        self._make_room(count, self.promised - promised)
        result = [self.free.pop() for _ in range(count)]
        for page in result:
            self.refs[page] = 1
        self.promised -= promised
        return result

    def promise(self, count):
        """Set COUNT free pages aside for later `allocate(..., promised=...)` calls."""
        if count < 0:
            raise ValueError("negative promise")
        self._make_room(count, self.promised)
        self.promised += count

    def unpromise(self, count):
        if count < 0 or count > self.promised:
            raise RuntimeError("promise underflow")
        self.promised -= count

    # ---- prefix index -------------------------------------------------
    def _keys(self, tokens, namespace):
        parent = hashlib.sha256(namespace.encode()).digest()
        size = self.page_size
        for start in range(0, len(tokens) - size + 1, size):
            chunk = tokens[start:start + size]
            parent = hashlib.sha256(parent + struct.pack(f"<{len(chunk)}q", *chunk)).digest()
            yield parent

    def acquire_prefix(self, tokens, namespace="local"):
        table = []
        if self.prefix_cache:
            # At least the last prompt token must run to recover its logits.
            for key in self._keys(tokens[:-1], namespace):
                page = self.prefixes.get(key)
                if page is None:
                    break
                self.prefixes.move_to_end(key)
                self.refs[page] += 1
                table.append(page)
        return table

    def publish(self, tokens, computed, table, namespace="local"):
        if not self.prefix_cache:
            return
        for i, key in enumerate(self._keys(tokens[:computed], namespace)):
            if key not in self.prefixes and table[i] >= 0:
                self.prefixes[key] = table[i]
                self.refs[table[i]] += 1

    def clear_prefixes(self):
        for page in self.prefixes.values():
            self._release_one(page)
        self.prefixes.clear()

    # ---- checks ---------------------------------------------------------
    def check(self, tables=()):
        """Raise if a page is lost, free and held at once, or counted wrongly.

        TABLES are the page lists of every live request of this group.
        """
        held = [0] * self.capacity
        for table in tables:
            for page in table:
                if page >= 0:
                    held[page] += 1
        for page in self.prefixes.values():
            held[page] += 1
        free = set(self.free)
        if len(free) != len(self.free):
            raise AssertionError("a page is on the free list twice")
        for page in range(self.capacity):
            if held[page] != self.refs[page]:
                raise AssertionError(f"page {page}: {self.refs[page]} references counted, {held[page]} held")
            if (page in free) != (self.refs[page] == 0):
                raise AssertionError(f"page {page} is {'free' if page in free else 'held'} with {self.refs[page]} references")
        if self.promised < 0 or self.promised > len(self.free):
            raise AssertionError("more pages promised than are free")
