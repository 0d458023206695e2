"""The cache manager on the host: no page lost, held twice or freed twice, under random orders of requests."""
import random

import pytest

from tessweave_engine_amd.cache import (CacheLayout, CacheManager, CacheNeed, CapacityError, FixedState, PagedKV,
                                        PagePool)
from tessweave_engine_amd.cache.pages import block_keys


def full_layout(layers=2):
    return CacheLayout([CacheNeed(PagedKV(2, 16))] * layers)


def test_pool_reference_vectors():
    # flow_engine tests/test_engine.py:149-158: eviction never gives away a page a request still holds.
    # (The reference drops the index entry on the failed attempt, refs == 1; here an attempt that cannot
    # succeed leaves the index alone, so the page keeps both uses.)
    p = PagePool(2, 4)
    table = p.allocate(1)
    p.publish([1, 2, 3, 4], 4, table)
    with pytest.raises(CapacityError):
        p.allocate(2)
    assert p.refs[table[0]] == 2 and len(p.prefixes) == 1 and p.evictions == 0
    p.release(table)
    assert len(p.allocate(2)) == 2 and not p.prefixes and p.evictions == 1
    # underflow and negative counts
    q = PagePool(2, 4)
    t = q.allocate(1)
    q.release(t)
    with pytest.raises(RuntimeError):
        q.release(t)
    with pytest.raises(ValueError):
        q.allocate(-1)


def test_prefix_keys_full_blocks_namespaces_and_last_token():
    p = PagePool(8, 4)
    table = p.allocate(3)
    tokens = [2, 3, 4, 5, 6, 7, 8, 9, 10]
    p.publish(tokens, 9, table)                        # two full blocks are keyed, the tail of one token is not
    assert len(p.prefixes) == 2
    assert p.acquire_prefix(tokens) == table[:2]       # cached == 8 of 9: the last token always runs
    assert p.acquire_prefix(tokens[:8]) == table[:1]   # lookup never covers the last prompt token
    assert p.acquire_prefix([2, 3, 4, 5, 60, 70]) == table[:1]          # divergent tail: one block shared
    assert p.acquire_prefix(tokens, namespace="tenant-b") == []
    assert p.refs[table[0]] == 1 + 1 + 3 and p.refs[table[1]] == 1 + 1 + 1
    off = PagePool(8, 4, prefix_cache=False)
    t2 = off.allocate(3)
    off.publish(tokens, 9, t2)
    assert off.acquire_prefix(tokens) == [] and not off.prefixes


def test_a_chain_published_portion_by_portion_is_still_eaten_from_its_tail():
    """The scheduler offers a prompt's blocks as its portions are issued, root first. The root must not
    be left the oldest entry: one eviction would then cut off every deeper block while they still hold pages."""
    tokens = [1, 2, 3, 4, 5, 6]
    p = PagePool(5, 2)
    a = p.allocate(3)
    for upto in (2, 4, 6):
        p.publish(tokens, upto, a)
    p.release(a)
    assert list(p.prefixes.values()) == [a[2], a[1], a[0]]          # deepest oldest, root youngest
    got = p.allocate(3)                                             # two pages are free, one must be evicted
    assert p.evictions == 1 and a[2] in got
    assert p.acquire_prefix(tokens + [7]) == a[:2]                  # what is left is reachable from the root
    # a block that a second request publishes again (same tokens) re-ages the chain, it does not duplicate it
    q = PagePool(6, 2)
    a = q.allocate(3)
    q.publish(tokens, 6, a)
    b = q.allocate(1)
    q.publish([9, 9], 2, b)
    q.publish(tokens, 4, a)                                         # the chain's first two blocks are young again
    q.release(a + b)
    assert list(q.prefixes.values()) == [a[2], b[0], a[1], a[0]]
    q.check()


def test_block_keys_go_on_from_known_keys_and_keep_the_format():
    import hashlib, struct
    tokens = list(range(100, 123))
    whole = block_keys(tokens, 4, "ns")
    assert len(whole) == 5
    root = hashlib.sha256(b"ns").digest()                           # flow_engine/cache.py:60-65
    first = hashlib.sha256(root + struct.pack("<4q", *tokens[:4])).digest()
    assert whole[0] == first
    assert whole[1] == hashlib.sha256(first + struct.pack("<4q", *tokens[4:8])).digest()
    assert block_keys(tokens, 4, "ns", known=whole[:2]) == whole
    assert block_keys(tokens[:9], 4, "ns", known=whole) == whole[:2]      # more known than asked for
    assert block_keys(tokens, 4, "other") != whole
    assert block_keys([-1, 5, 2 ** 40, 0], 4, "ns")[0] == hashlib.sha256(root + struct.pack("<4q", -1, 5, 2 ** 40, 0)).digest()


def test_manager_hashes_each_block_of_a_request_once(monkeypatch):
    import tessweave_engine_amd.cache.manager as manager_module
    hashed = []
    real = manager_module.block_keys

    def counting(tokens, page_size, namespace, known=()):
        hashed.append(len(tokens) // page_size - min(len(known), len(tokens) // page_size))
        return real(tokens, page_size, namespace, known)

    monkeypatch.setattr(manager_module, "block_keys", counting)
    m = CacheManager(full_layout(), page_size=4, pages=16, max_requests=2, max_request_tokens=64)
    prompt = list(range(40))
    a = m.open("a")
    assert m.acquire_prefix(a, prompt) == 0                         # hashes the 9 blocks a lookup may use
    for upto in (8, 16, 24, 40):
        m.ensure(a, upto)
        m.advance(a, upto)
        m.publish(a, prompt, computed=upto)
    m.publish(a, prompt + [1, 2, 3, 4], computed=40)                # the finished sequence: nothing new below 40
    assert sum(hashed) == 10                                        # 40 tokens, 10 blocks, each hashed once
    b = m.open("b")
    assert m.acquire_prefix(b, prompt) == 36
    assert m.acquire_prefix(b, prompt) == 0                         # a request that holds pages takes no more
    m.close(a), m.close(b)
    m.check()


def test_eviction_takes_unused_entries_oldest_first_and_a_chain_from_its_tail():
    p = PagePool(6, 2)
    a = p.allocate(3)
    p.publish([1, 2, 3, 4, 5, 6], 6, a)                 # one chain of three blocks
    b = p.allocate(1)
    p.publish([9, 9], 2, b)                             # a younger, unrelated entry
    p.release(a + b)
    assert len(p.free) == 2 and p.available() == 6
    held = p.acquire_prefix([1, 2, 7])                  # touches the chain's root and pins its page
    assert held == a[:1]
    got = p.allocate(4)                                 # needs two evictions: the chain's tail goes first
    assert p.evictions == 2 and set(got) >= {a[2], a[1]}
    assert p.acquire_prefix([1, 2, 3]) == a[:1] and p.acquire_prefix([9, 9, 0]) == b
    # a request that cannot be satisfied even by evicting everything leaves the index as it is
    before = list(p.prefixes)
    with pytest.raises(CapacityError):
        p.allocate(3)
    assert list(p.prefixes) == before
    p.check([got, held, a[:1], b])


def test_promises_set_pages_aside():
    p = PagePool(4, 4)
    p.promise(3)
    with pytest.raises(CapacityError):
        p.allocate(2)                                   # only one page is unpromised
    mine = p.allocate(2, promised=2)
    assert p.promised == 1 and len(p.free) == 2
    other = p.allocate(1)
    with pytest.raises(CapacityError):
        p.promise(1)
    p.release(mine + other)
    p.unpromise(1)
    p.check()
    assert len(p.free) == 4


def test_window_group_returns_pages_as_the_window_passes():
    layout = CacheLayout([CacheNeed(PagedKV(2, 16)), CacheNeed(PagedKV(2, 16, window=8))])
    assert len(layout.groups) == 2 and not layout.shares_prefixes
    m = CacheManager(layout, 4, [16, 5], 2, max_request_tokens=64)
    s = m.open("a")
    for upto in range(1, 61):
        m.ensure(s, upto)
        m.advance(s, upto)
        m.check()
        held = s.held(1)
        assert held <= m.pages_needed(1, 64, 1), (upto, held)           # 8 keys + 1 token: at most 3 pages of 4
        first = max(0, upto - 8 + 1) // 4
        assert s.tables[1][:first] == [-1] * first and all(p >= 0 for p in s.tables[1][first:])
    assert s.held(0) == 15
    m.close(s)
    m.check()
    assert all(len(p.free) == p.capacity for p in m.pools)


def test_reservation_for_windows_counts_the_largest_step():
    layout = CacheLayout([CacheNeed(PagedKV(1, 16, window=16))])
    m = CacheManager(layout, 4, 8, 2, max_request_tokens=256)
    assert m.pages_needed(0, 256, 1) == 5 and m.pages_needed(0, 256, 13) == 8 and m.pages_needed(0, 10, 13) == 3
    s = m.open("a")
    m.reserve(s, 200, largest_step=13)
    assert m.pools[0].promised == 8
    other = m.open("b")
    with pytest.raises(CapacityError):
        m.reserve(other, 10, 13)
    done = 0
    for step in [13, 13, 1, 1, 13, 7, 1, 13, 13, 13, 1, 1, 1, 13]:
        m.ensure(s, done + step)
        done += step
        m.advance(s, done)
        m.check()
        assert s.held(0) + s.promised[0] == 8
    m.close(s)
    m.reserve(other, 10, 13)
    m.close(other)
    m.check()
    assert m.pools[0].promised == 0 and len(m.pools[0].free) == 8


def test_state_slots_and_request_limit():
    layout = CacheLayout([CacheNeed(PagedKV(2, 16), FixedState((3, 5))), CacheNeed(state=FixedState((7,), "int32"))])
    assert layout.state_slots == (0, 1) and len(layout.groups) == 1 and not layout.shares_prefixes
    m = CacheManager(layout, 4, 8, 2)
    a, b = m.open("a"), m.open("b")
    assert {a.state_slot, b.state_slot} == {0, 1}
    with pytest.raises(CapacityError):
        m.open("c")
    with pytest.raises(ValueError):
        m.open("a")
    m.close(a)
    with pytest.raises(RuntimeError):
        m.close(a)
    c = m.open("c")
    assert c.state_slot == a.state_slot
    m.check()


def test_prefix_reuse_through_the_manager():
    m = CacheManager(full_layout(), 4, 16, 4, max_request_tokens=32)
    assert m.prefix_cache
    prompt = [2, 3, 4, 5, 6, 7, 8, 9, 10]
    a = m.open("a")
    assert m.acquire_prefix(a, prompt) == 0
    m.ensure(a, 9)
    m.advance(a, 9)
    m.publish(a, prompt)
    m.close(a)
    m.check()
    b = m.open("b")
    assert m.acquire_prefix(b, prompt) == 8 and b.computed == 8 and b.cached == 8
    m.ensure(b, 9)
    assert b.tables[0][:2] == a.tables[0][:2] if a.tables[0] else True
    m.check()
    m.close(b)
    m.clear_prefixes()
    m.check()
    assert len(m.pools[0].free) == 16


@pytest.mark.parametrize("seed", range(12))
def test_random_orders_of_requests(seed):
    rng = random.Random(seed)
    windowed = seed % 3 == 0
    needs = [CacheNeed(PagedKV(2, 16)), CacheNeed(PagedKV(2, 16, window=6) if windowed else PagedKV(2, 16))]
    m = CacheManager(CacheLayout(needs), 4, [12, 9] if windowed else 12, 4, max_request_tokens=40)
    live, tokens, counter = {}, {}, 0
    for _ in range(400):
        action = rng.random()
        if action < 0.25 and len(live) < 4:
            rid = f"r{counter}"
            counter += 1
            seq = m.open(rid)
            if not windowed:
                prompt = [rng.randrange(3) for _ in range(rng.randrange(1, 14))]
                m.acquire_prefix(seq, prompt)
                tokens[rid] = prompt
            live[rid] = seq
        elif action < 0.8 and live:
            rid = rng.choice(sorted(live))
            seq = live[rid]
            grow = rng.choice([1, 1, 1, 2, 3, 5])
            try:
                m.ensure(seq, min(40, seq.computed + grow))
                m.advance(seq, min(40, seq.computed + grow))
            except CapacityError:
                pass                                        # nothing may have changed
        elif live:
            rid = rng.choice(sorted(live))
            seq = live.pop(rid)
            if not windowed and rng.random() < 0.6:
                history = (tokens[rid] + [1] * 40)[:seq.computed]
                m.publish(seq, history)
            m.close(seq)
        m.check()
    for seq in live.values():
        m.close(seq)
    m.clear_prefixes()
    m.check()
    assert all(len(p.free) == p.capacity and p.promised == 0 for p in m.pools)
    assert sorted(m.free_state_slots) == [0, 1, 2, 3]


def test_ensure_is_all_or_nothing_across_groups():
    layout = CacheLayout([CacheNeed(PagedKV(2, 16)), CacheNeed(PagedKV(1, 32))])
    m = CacheManager(layout, 4, [8, 2], 2, max_request_tokens=32)
    s = m.open("a")
    m.ensure(s, 8)
    with pytest.raises(CapacityError):
        m.ensure(s, 12)                                  # group 1 has no third page
    m.check()
    assert s.held(0) == 2 and s.held(1) == 2 and len(m.pools[0].free) == 6
    with pytest.raises(ValueError):
        m.ensure(s, 33)
    assert m.slot_of(s, 0, 5) == s.tables[0][1] * 4 + 1


def test_slot_arithmetic_vector_of_the_reference():
    """docs/ARCHITECTURE.md:51-53 of the reference: position 37, pages of 16, table[2] = 7 -> slot 117."""
    m = CacheManager(full_layout(), 16, 9, 2, max_request_tokens=48)
    seq = m.open("r")
    m.pools[0].free = [0, 8, 6, 5, 4, 3, 7, 2, 1]            # pages come off the end: 1, 2, then 7
    m.ensure(seq, 38)
    assert seq.tables[0] == [1, 2, 7]
    assert m.slot_of(seq, 0, 37) == 117 and m.slot_of(seq, 0, 0) == 16 and m.slot_of(seq, 0, 31) == 47
    assert m.table_rows[0][seq.state_slot].tolist() == [1, 2, 7]
    m.close(seq)
    m.check()
