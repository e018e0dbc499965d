"""The cache manager on the CPU: no page lost, held twice or freed twice, under random orders
of requests; windows give pages back; prefix reuse; state slots. Includes the reference's own
test vectors (tests/test_block_manager.py:7-28 of the reference, read with prefix caching on)."""
import random

import pytest

from minivllm_amd.cache import (CacheManager, GroupSpec, OutOfPages, OutOfSlots, PagePool, StateSlots, page_hash)
from minivllm_amd.parts import KeepAll, KeepWindow, Retention

from dataclasses import dataclass


@dataclass(frozen=True)
class KeepChunk(Retention):
    """A third rule, defined here: a query sees the positions of its own chunk of ``chunk`` tokens
    only, so every page before the chunk of the next query can go."""
    chunk: int = 1

    def first_kept_page(self, next_position, page_size):
        return (next_position // self.chunk) * self.chunk // page_size


FULL = GroupSpec(KeepAll(), (0, 1))
WIN = GroupSpec(KeepWindow(21), (2,))
CHUNK = GroupSpec(KeepChunk(12), (3,))


def test_page_hash_is_the_references_chain():
    """xxh64 over the previous hash as 8 bytes LE, then each token as 4 bytes LE signed
    (minivllm/kvcache/block_manager.py:24-30)."""
    import xxhash
    toks = [5, 70000, 0, 2 ** 31 - 1]
    h = xxhash.xxh64()
    for t in toks:
        h.update(t.to_bytes(4, "little", signed=True))
    assert page_hash(toks) == h.intdigest()
    h2 = xxhash.xxh64()
    h2.update(h.intdigest().to_bytes(8, "little"))
    for t in toks:
        h2.update(t.to_bytes(4, "little", signed=True))
    assert page_hash(toks, h.intdigest()) == h2.intdigest()
    assert page_hash(toks, h.intdigest()) != page_hash(toks)


def test_reference_vectors_with_prefix_caching():
    ps = 256
    m = CacheManager([GroupSpec(KeepAll(), (0,))], 10240, ps, 512, enable_prefix_caching=True)
    rng = random.Random(0)
    tokens = [rng.randint(1, 25600) for _ in range(25600)]
    m.admit("big", tokens)
    m.reserve("big", len(tokens))
    m.commit("big", len(tokens), tokens)
    assert len(m.block_table("big", 0)) == 100
    assert m.pools[0].num_hashed == 100 and m.pools[0].num_used == 100
    live = []
    for i in range(1, 100):
        rid = f"r{i}"
        prompt = tokens[:i * ps]
        seq = m.admit(rid, prompt)
        # every full page but the last is found; the last is left so that one token is computed
        assert seq.num_computed == (i - 1) * ps == seq.num_cached
        rest = len(prompt) - seq.num_computed
        if not m.can_reserve(rid, rest):
            m.release(rid)
            for r in live:
                m.release(r)
            live.clear()
            seq = m.admit(rid, prompt)
        m.reserve(rid, rest)
        m.commit(rid, rest, prompt)
        assert len(m.block_table(rid, 0)) == i
        assert m.block_table(rid, 0)[:i - 1] == m.block_table("big", 0)[:i - 1]
        live.append(rid)
        m.check_invariants()


def test_pool_fifo_and_double_free():
    pool = PagePool(3)
    a, b, c = pool.allocate(), pool.allocate(), pool.allocate()
    assert (a, b, c) == (0, 1, 2)
    with pytest.raises(OutOfPages):
        pool.allocate()
    pool.release(b); pool.release(a)
    assert pool.allocate() == b                   # the page that has been free longest goes first
    with pytest.raises(AssertionError):
        pool.release(c); pool.release(c)
    pool.check()


def test_hash_hit_needs_equal_tokens_and_entries_do_not_leak():
    pool = PagePool(2)
    p = pool.allocate()
    pool.publish(p, 123, [1, 2, 3])
    assert pool.lookup(123, [1, 2, 3]) == p
    assert pool.lookup(123, [1, 2, 4]) is None    # same hash, other tokens (block_manager.py:69)
    pool.release(p)
    assert pool.lookup(123, [1, 2, 3]) == p       # a freed page keeps its content until reused
    q = pool.allocate(); r = pool.allocate()
    assert {q, r} == {0, 1}
    assert pool.lookup(123, [1, 2, 3]) is None and pool.num_hashed == 0


def test_window_group_gives_pages_back():
    ps = 8
    m = CacheManager([FULL, WIN], 64, ps, 4)
    m.admit("a")
    for n in (7, 5, 30, 1, 1, 40):
        m.reserve("a", n)
        m.commit("a", n)
        seq = m.sequence("a")
        computed = seq.num_computed
        full, win = seq.pages
        assert all(p >= 0 for p in full) and len(full) == -(-computed // ps)
        first_kept = max(0, computed - 21) // ps      # the next query at `computed` sees positions >= computed-21
        assert all(p == -1 for p in win[:first_kept]) and all(p >= 0 for p in win[first_kept:])
        m.check_invariants()
    assert m.pools[1].num_used <= -(-(21 + 1) // ps) + 1
    m.release("a")
    assert m.pools[0].num_free == 64 and m.pools[1].num_free == 64


def test_a_retention_rule_defined_outside_the_framework():
    """The manager asks a group's retention object for the first page still needed and nothing else:
    a rule defined in this file (the chunk of the next query) gives its pages back like the others."""
    ps = 8
    m = CacheManager([FULL, CHUNK], 64, ps, 4)
    assert [g.retention.key() for g in m.groups] == [("KeepAll",), ("KeepChunk", ("chunk", 12))]
    m.admit("a")
    for n in (7, 5, 30, 1, 1, 40, 11):
        m.reserve("a", n)
        m.commit("a", n)
        seq = m.sequence("a")
        first_kept = (seq.num_computed // 12) * 12 // ps
        kept = seq.pages[1]
        assert all(p == -1 for p in kept[:first_kept]) and all(p >= 0 for p in kept[first_kept:])
        assert all(p >= 0 for p in seq.pages[0])
        m.check_invariants()
    assert m.pools[1].num_used <= 3
    m.release("a")
    assert all(p.num_free == 64 for p in m.pools)
    with pytest.raises(TypeError):
        GroupSpec("full", (0,))                      # a name is not a rule


def test_reserve_is_all_or_nothing():
    m = CacheManager([FULL, WIN], [10, 2], 4, 4)
    m.admit("a")
    with pytest.raises(OutOfPages):
        m.reserve("a", 12)                            # the window pool has 2 pages only
    assert m.pools[0].num_free == 10 and m.pools[1].num_free == 2
    assert m.reservable_tokens("a") == 8
    m.reserve("a", 8)
    m.commit("a", 8)
    m.check_invariants()


def test_state_slots():
    s = StateSlots(2)
    a, b = s.take(), s.take()
    assert {a, b} == {0, 1}
    with pytest.raises(OutOfSlots):
        s.take()
    s.release(a)
    assert s.take() == a
    with pytest.raises(AssertionError):
        s.release(5)
    m = CacheManager([FULL], 8, 4, 2)
    m.admit("x"); m.admit("y")
    assert not m.can_admit()
    assert m.sequence("x").state_slot != m.sequence("y").state_slot
    m.release("x")
    assert m.can_admit()
    m.admit("z")
    m.check_invariants()


@pytest.mark.parametrize("seed", range(6))
@pytest.mark.parametrize("prefix", [False, True])
def test_random_orders(seed, prefix):
    """Random admissions, portions, decodes, preemptions and ends; the books balance after
    every operation and every page is back at the end."""
    rng = random.Random(seed)
    ps = rng.choice([4, 8, 16])
    groups = [FULL] if prefix else [FULL, WIN, CHUNK]
    m = CacheManager(groups, 40, ps, 6, enable_prefix_caching=prefix)
    assert m.prefix_caching == prefix
    shared = [rng.randrange(100) for _ in range(3 * ps)]
    live = {}
    next_id = 0
    for _ in range(600):
        op = rng.random()
        if op < 0.2 and m.can_admit():
            toks = (shared if rng.random() < 0.5 else []) + [rng.randrange(100) for _ in range(rng.randint(1, 50))]
            rid = next_id; next_id += 1
            seq = m.admit(rid, toks)
            assert seq.num_computed <= len(toks) - 1 and seq.num_computed % ps == 0
            live[rid] = toks
        elif op < 0.85 and live:
            rid = rng.choice(list(live))
            toks = live[rid]
            left = len(toks) - m.sequence(rid).num_computed
            if left == 0:
                toks.append(rng.randrange(100)); left = 1       # a decoded token
            n = rng.randint(1, left)
            if m.can_reserve(rid, n):
                m.reserve(rid, n)
                m.commit(rid, n, toks)
            else:
                victim = rng.choice(list(live))                  # preempt someone
                m.release(victim); del live[victim]
        elif live:
            rid = rng.choice(list(live))
            m.release(rid); del live[rid]
        m.check_invariants()
    for rid in list(live):
        m.release(rid)
    m.check_invariants()
    assert all(p.num_free == p.num_pages for p in m.pools) and m.slots.num_free == 6


def test_prefix_reuse_is_off_with_windows_or_state():
    assert not CacheManager([FULL, WIN], 8, 4, 2, enable_prefix_caching=True).prefix_caching
    assert not CacheManager([FULL], 8, 4, 2, enable_prefix_caching=True, has_state=True).prefix_caching
    assert CacheManager([FULL], 8, 4, 2, enable_prefix_caching=True).prefix_caching
