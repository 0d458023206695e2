"""What a mixer asks of the cache, and how the layers' needs are grouped.

The reference keeps one uniform pool `[L, blocks, block_size, Hkv, D]` for all
layers (flow_engine/cache.py:21) and no per-request state. Here every cache
slot (one per layer run that writes a cache) declares its need; slots with the
same paged need share one GROUP: one page pool, one block table per request. A
slot may also (or instead) ask for a fixed-size state per request.
"""
from __future__ import annotations

from dataclasses import dataclass


@dataclass(frozen=True)
class PagedKV:
    """Keys and values of every token (window None) or of the last `window` tokens."""
    kv_heads: int
    head_dim: int
    window: int | None = None

    def __post_init__(self):
        if self.kv_heads <= 0 or self.head_dim <= 0:
            raise ValueError("kv_heads and head_dim must be positive")
        if self.window is not None and self.window <= 0:
            raise ValueError("a window must be positive (None means all keys)")


@dataclass(frozen=True)
class FixedState:
    """State of fixed size per request, e.g. a recurrent mixer's."""
    shape: tuple
    dtype: str = "float32"

    def __post_init__(self):
        object.__setattr__(self, "shape", tuple(int(s) for s in self.shape))
        if any(s <= 0 for s in self.shape):
            raise ValueError("state dimensions must be positive")
        if self.dtype not in ("float32", "bfloat16", "int32"):
            raise ValueError("state dtype must be float32, bfloat16 or int32")


@dataclass(frozen=True)
class CacheNeed:
    paged: PagedKV | None = None
    state: FixedState | None = None


@dataclass(frozen=True)
class CacheGroup:
    spec: PagedKV
    slots: tuple          # cache slots stored in this group, in storage order


class CacheLayout:
    """Cache slots of a model, grouped by paged need."""

    def __init__(self, needs):
        self.needs = tuple(needs)
        groups: dict[PagedKV, list[int]] = {}
        for slot, need in enumerate(self.needs):
            if need is not None and need.paged is not None:
                groups.setdefault(need.paged, []).append(slot)
        self.groups = tuple(CacheGroup(spec, tuple(slots)) for spec, slots in groups.items())
        self.slot_group = {}
        for g, group in enumerate(self.groups):
            for i, slot in enumerate(group.slots):
                self.slot_group[slot] = (g, i)
        self.state_slots = tuple(slot for slot, need in enumerate(self.needs)
                                 if need is not None and need.state is not None)

    @property
    def shares_prefixes(self):
        """Full pages of a prompt prefix can be reused only if they are all a request holds."""
        return (len(self.groups) == 1 and self.groups[0].spec.window is None
                and not self.state_slots)

    def bytes_per_token(self, element_bytes):
        return sum(2 * len(g.slots) * g.spec.kv_heads * g.spec.head_dim * element_bytes
                   for g in self.groups)
