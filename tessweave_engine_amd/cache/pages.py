"""Who owns which physical page of one cache group (host side only; no tensors here).

A page carries a use count: one for every live request whose block table names
it and one if the prefix index names it. It is on the free list exactly while
that count is zero. Requests may also be PROMISED pages: a promise sets free
pages aside without choosing them, and is redeemed page by page as the request
grows, so a request admitted with a promise for its worst case can never be
starved by later arrivals.

The prefix index maps the key of a FULL block of tokens to the page that holds
its keys and values. The key format is a contract shared with the reference
(flow_engine/cache.py:60-65): the root is sha256(namespace), and every block's
key is sha256(parent key + the block's token ids as little-endian int64), so a
key names the whole prefix up to and including its block. What the reference
fixes besides the format: lookups never cover a prompt's last token, whose
logits must be computed (cache.py:69-70); a hit refreshes an entry's age
(cache.py:75); pages come off the free list last-in first-out (cache.py:25,55);
a use count below zero is an error (cache.py:36-37).

Eviction differs from the reference's (cache.py:49-54), which pops entries
oldest first whether or not that frees anything and so can empty the index on
behalf of a request that then still does not fit. Here a request for pages is
first checked against what eviction COULD free; only then are entries dropped,
oldest first, and only entries whose page nobody else uses. Within one prefix
chain deeper blocks are kept older than their parents, so a chain is eaten from
its tail and what stays is still reachable from the root. Both a lookup and a
publication re-age the whole chain they walk, root last: a chain that enters
the index portion by portion (its root first) keeps that order too.
"""
from __future__ import annotations

from collections import OrderedDict
import hashlib
import struct


class CapacityError(RuntimeError):
    """Not enough free pages (or state slots); the caller waits or refuses."""


def block_keys(tokens, page_size, namespace, known=()):
    """Keys of the full blocks of TOKENS, root first.

    KNOWN: the keys of the first len(KNOWN) blocks, if the caller already has them (a key names its
    whole prefix, so hashing goes on from the last of them and touches only the blocks after it).
    """
    keys = list(known[:len(tokens) // page_size])
    key = keys[-1] if keys else hashlib.sha256(namespace.encode()).digest()
    pack = struct.Struct("<%dq" % page_size).pack
    for end in range((len(keys) + 1) * page_size, len(tokens) + 1, page_size):
        key = hashlib.sha256(key + pack(*tokens[end - page_size:end])).digest()
        keys.append(key)
    return keys


class PagePool:
    def __init__(self, pages, page_size, prefix_cache=True):
        if pages <= 0 or page_size <= 0:
            raise ValueError("pages and page_size must be positive")
        self.capacity = int(pages)
        self.page_size = int(page_size)
        self.refs = [0] * self.capacity                       # use count per page
        self.free = list(range(self.capacity - 1, -1, -1))    # a stack: page 0 is handed out first
        self.prefixes: OrderedDict[bytes, int] = OrderedDict()   # block key -> page, oldest entry first
        self.prefix_cache = bool(prefix_cache)
        self.promised = 0
        self.hits = 0            # prompt tokens served from the index (counted by whoever admits the request)
        self.evictions = 0

    # ---- use counts -------------------------------------------------------------------
    def _use(self, page):
        self.refs[page] += 1

    def _unuse(self, page):
        if not 0 <= page < self.capacity:
            raise RuntimeError(f"page id {page} out of range")
        left = self.refs[page] - 1
        if left < 0:
            raise RuntimeError("KV reference underflow")
        self.refs[page] = left
        if left == 0:
            self.free.append(page)

    def release(self, pages):
        """Drop one use of every page in PAGES (-1 marks a block that is not held)."""
        for page in pages:
            if page >= 0:
                self._unuse(page)

    # ---- free pages, promises, eviction -------------------------------------------------
    def _index_only(self):
        """Keys, oldest first, of entries whose page only the index uses."""
        return [key for key, page in self.prefixes.items() if self.refs[page] == 1]

    def available(self):
        """Pages that a new promise or an unpromised allocation could still get."""
        return len(self.free) + len(self._index_only()) - self.promised

    def _free_up(self, count, set_aside):
        """Make COUNT pages free beyond the SET_ASIDE ones that stay promised to others.

        Raises CapacityError, and leaves the index as it is, if eviction could not free enough.
        """
        short = count + set_aside - len(self.free)
        if short <= 0:
            return
        victims = self._index_only()
        if len(victims) < short:
            raise CapacityError("KV capacity exhausted; request must wait or reduce its token budget")
        for key in victims[:short]:
            self._unuse(self.prefixes.pop(key))
            self.evictions += 1

    def allocate(self, count, promised=0):
        """Take COUNT pages; PROMISED of them redeem a promise made before."""
        if count < 0 or not 0 <= promised <= min(count, self.promised):
            raise ValueError("negative allocation")
        self._free_up(count, self.promised - promised)
        self.promised -= promised
        taken = [self.free.pop() for _ in range(count)]
        for page in taken:
            self.refs[page] = 1
        return taken

    def promise(self, count):
        """Set COUNT pages aside for later `allocate(..., promised=...)` calls."""
        if count < 0:
            raise ValueError("negative promise")
        self._free_up(count, self.promised)
        self.promised += count

    def unpromise(self, count):
        if not 0 <= count <= self.promised:
            raise RuntimeError("promise underflow")
        self.promised -= count

    # ---- prefix index -------------------------------------------------------------------
    def acquire_prefix(self, tokens, namespace="local", keys=None):
        """Pages of the longest indexed prefix of TOKENS, each with one more use; never the last token's block.
        KEYS: the block keys of TOKENS, if the caller has them."""
        if not self.prefix_cache:
            return []
        usable = (len(tokens) - 1) // self.page_size
        if keys is None:
            keys = block_keys(tokens[:usable * self.page_size], self.page_size, namespace)
        found = []
        for key in keys[:usable]:
            page = self.prefixes.get(key)
            if page is None:
                break
            found.append((key, page))
        for key, page in reversed(found):       # the root ends up youngest, the deepest block oldest of the chain
            self.prefixes.move_to_end(key)
            self._use(page)
        return [page for _, page in found]

    def publish(self, tokens, computed, table, namespace="local", keys=None):
        """Enter the full blocks of TOKENS[:COMPUTED] (pages TABLE[i]) that the index does not know yet.
        KEYS: the block keys of TOKENS[:COMPUTED], if the caller has them.

        The whole chain is re-aged, deepest block first and root last, whether its blocks are new to the
        index or not: a prompt that is published portion by portion would otherwise leave its root the
        oldest entry, and one eviction would cut every deeper block off.
        """
        if not self.prefix_cache:
            return
        blocks = int(computed) // self.page_size
        if keys is None:
            keys = block_keys(tokens[:blocks * self.page_size], self.page_size, namespace)
        for i in range(min(blocks, len(keys)) - 1, -1, -1):
            key = keys[i]
            if key in self.prefixes:
                self.prefixes.move_to_end(key)
            elif table[i] >= 0:
                self.prefixes[key] = table[i]
                self._use(table[i])

    def clear_prefixes(self):
        while self.prefixes:
            self._unuse(self.prefixes.popitem()[1])

    # ---- checks ---------------------------------------------------------------------------
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
        if not 0 <= self.promised <= len(self.free):
            raise AssertionError("more pages promised than are free")
