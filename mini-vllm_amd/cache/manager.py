"""The cache manager: pages of keys and values with a block table per request, for groups of
calls with different retention, and a state slot per request.

Reference: minivllm/kvcache/block_manager.py manages one uniform pool for all layers and
allocates a whole prompt at once (block_manager.py:54-87) or one page per decode step
(block_manager.py:89-98). Here

* calls (layer executions) whose mixers need the same retention form a *group*; each group has
  its own pool and each request one block table per group. How long a group keeps a position is
  its ``Retention`` object's business (``parts.base``): the manager asks it only for the first page
  a request still needs (``KeepAll`` keeps every position; ``KeepWindow`` gives a page back as soon
  as every position in it lies more than ``window`` tokens behind the next query; a mixer with
  another rule brings its own class);
* pages are reserved for the portion of tokens about to run (``reserve``), and the request's
  progress is recorded after the step (``commit``), which also publishes pages that became full
  for prefix reuse and returns pages a window has passed;
* prefix reuse (``enable_prefix_caching``) is offered when every group keeps all positions
  (``Retention.keeps_everything``) and no call carries state, and never covers the whole prompt: at least one token is left to
  compute (in the reference a full hit leaves no query at all);
* a request holds one state slot from ``admit`` to ``release``.

The manager is host-side bookkeeping only; it never touches device memory.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Dict, Hashable, List, Optional, Sequence, Tuple

import numpy as np

from ..parts.base import Retention
from .page_pool import OutOfPages, PagePool, page_hash
from .state_slots import StateSlots


@dataclass(frozen=True)
class GroupSpec:
    """One cache group: the calls it serves and how long it keeps a position."""
    retention: Retention
    calls: Tuple[int, ...]

    def __post_init__(self):
        if not isinstance(self.retention, Retention):
            raise TypeError(f"a cache group's retention must be a Retention object, got {self.retention!r}")


def groups_from_needs(needs: Sequence[Optional[object]]) -> List[GroupSpec]:
    """Groups the calls by what their mixers need (``CacheNeed.group_key()``); calls without a
    need are in no group."""
    keyed: Dict[Tuple, List[int]] = {}
    rules: Dict[Tuple, Retention] = {}
    for call, need in enumerate(needs):
        if need is None:
            continue
        key = need.group_key()
        keyed.setdefault(key, []).append(call)
        rules.setdefault(key, need.retention)
    return [GroupSpec(retention=rules[k], calls=tuple(v)) for k, v in keyed.items()]


@dataclass
class SequenceCache:
    """What one request holds."""
    state_slot: int
    pages: List[List[int]]            # per group: page id per page index, -1 once given back
    num_computed: int = 0             # positions whose keys and values are in the cache
    num_cached: int = 0               # of those, how many came from prefix reuse
    hashes: List[int] = field(default_factory=list)   # chained hashes of the full pages so far
    # the same page ids as int32 arrays (grown in steps), so that a step's block tables are copied
    # rather than converted element by element
    arrays: List[np.ndarray] = field(default_factory=list)

    def push(self, group: int, page: int) -> None:
        pages = self.pages[group]
        while len(self.arrays) <= group:
            self.arrays.append(np.full(16, -1, dtype=np.int32))
        arr = self.arrays[group]
        if len(pages) >= arr.size:
            grown = np.full(2 * arr.size, -1, dtype=np.int32)
            grown[:arr.size] = arr
            arr = self.arrays[group] = grown
        arr[len(pages)] = page
        pages.append(page)

    def drop(self, group: int, index: int) -> None:
        self.pages[group][index] = -1
        self.arrays[group][index] = -1

    def table(self, group: int) -> np.ndarray:
        """The block table of a group as an int32 array (a view: copy it before the next change)."""
        n = len(self.pages[group])
        if len(self.arrays) <= group:
            return np.empty(0, dtype=np.int32)
        return self.arrays[group][:n]


class CacheManager:
    def __init__(self, groups: Sequence[GroupSpec], num_pages, page_size: int, num_state_slots: int,
                 enable_prefix_caching: bool = False, has_state: bool = False):
        if page_size < 1:
            raise ValueError(f"page_size must be >= 1, got {page_size}")
        self.groups = list(groups)
        if isinstance(num_pages, int):
            num_pages = [num_pages] * len(self.groups)
        if len(num_pages) != len(self.groups):
            raise ValueError("one page count per group is needed")
        self.page_size = page_size
        self.pools = [PagePool(n) for n in num_pages]
        self.slots = StateSlots(num_state_slots)
        self.seqs: Dict[Hashable, SequenceCache] = {}
        self.prefix_caching = bool(enable_prefix_caching and self.groups and not has_state
                                   and all(g.retention.keeps_everything for g in self.groups))

    # ---- queries ----------------------------------------------------------------------------
    def __contains__(self, req) -> bool:
        return req in self.seqs

    def sequence(self, req) -> SequenceCache:
        return self.seqs[req]

    def num_free_pages(self, group: int = 0) -> int:
        return self.pools[group].num_free

    def _first_kept_page(self, g: int, next_position: int) -> int:
        """Index of the first page group ``g`` still needs when the next query stands at
        ``next_position``."""
        return self.groups[g].retention.first_kept_page(next_position, self.page_size)

    def pages_needed(self, req, num_new_tokens: int) -> List[int]:
        """Per group, how many pages must be allocated so that ``num_new_tokens`` more positions
        fit."""
        seq = self.seqs[req]
        total = -(-(seq.num_computed + num_new_tokens) // self.page_size)
        return [max(0, total - len(seq.pages[g])) for g in range(len(self.groups))]

    def reservable_tokens(self, req) -> int:
        """How many more positions the request could be given right now: room left in its last
        pages plus what the free pages of the tightest group hold."""
        seq = self.seqs[req]
        room = min((len(seq.pages[g]) + self.pools[g].num_free) * self.page_size
                   for g in range(len(self.groups))) if self.groups else 1 << 60
        return max(0, room - seq.num_computed)

    def fits(self, req, num_new_tokens: int) -> bool:
        """Whether the pages the request already holds take that many more positions."""
        seq = self.seqs[req]
        end = seq.num_computed + num_new_tokens
        ps = self.page_size
        for pages in seq.pages:
            if end > len(pages) * ps:
                return False
        return True

    def can_reserve(self, req, num_new_tokens: int) -> bool:
        return all(n <= self.pools[g].num_free for g, n in enumerate(self.pages_needed(req, num_new_tokens)))

    # ---- life of a request --------------------------------------------------------------------
    def can_admit(self) -> bool:
        return self.slots.num_free > 0

    def admit(self, req, tokens: Optional[Sequence[int]] = None) -> SequenceCache:
        """Registers a request, takes its state slot and, with prefix reuse on, shares the pages
        that already hold the leading full pages of ``tokens``. Returns its record;
        ``num_computed`` tells how many leading tokens need not be run."""
        if req in self.seqs:
            raise KeyError(f"request {req!r} is already admitted")
        slot = self.slots.take()
        seq = SequenceCache(state_slot=slot, pages=[[] for _ in self.groups])
        self.seqs[req] = seq
        if self.prefix_caching and tokens is not None:
            ps = self.page_size
            usable = (len(tokens) - 1) // ps          # leave at least one token to compute
            prefix: Optional[int] = None
            for i in range(usable):
                chunk = tokens[i * ps:(i + 1) * ps]
                h = page_hash(chunk, prefix)
                found = [pool.lookup(h, chunk) for pool in self.pools]
                if any(p is None for p in found):
                    break
                for g, p in enumerate(found):
                    self.pools[g].share(p)
                    seq.push(g, p)
                seq.hashes.append(h)
                prefix = h
                seq.num_computed += ps
            seq.num_cached = seq.num_computed
        return seq

    def reserve(self, req, num_new_tokens: int) -> None:
        """Allocates the pages that positions ``num_computed .. num_computed + n - 1`` need, in
        every group. Raises OutOfPages (and allocates nothing) when a pool is too small."""
        needed = self.pages_needed(req, num_new_tokens)
        for g, n in enumerate(needed):
            if n > self.pools[g].num_free:
                raise OutOfPages(f"group {g} needs {n} pages, {self.pools[g].num_free} are free")
        seq = self.seqs[req]
        for g, n in enumerate(needed):
            for _ in range(n):
                seq.push(g, self.pools[g].allocate())

    def commit(self, req, num_new_tokens: int, tokens: Optional[Sequence[int]] = None) -> None:
        """Records that the step wrote ``num_new_tokens`` more positions. ``tokens`` (the
        request's tokens from position 0, at least up to the new length) lets full pages be
        published for reuse."""
        seq = self.seqs[req]
        new_len = seq.num_computed + num_new_tokens
        ps = self.page_size
        for g in range(len(self.groups)):
            if new_len > len(seq.pages[g]) * ps:
                raise AssertionError(f"request {req!r}: {new_len} positions but only {len(seq.pages[g])} pages "
                                     f"in group {g}; reserve() first")
        if self.prefix_caching and tokens is not None:
            while (len(seq.hashes) + 1) * ps <= new_len:
                i = len(seq.hashes)
                chunk = tokens[i * ps:(i + 1) * ps]
                h = page_hash(chunk, seq.hashes[-1] if seq.hashes else None)
                for g, pool in enumerate(self.pools):
                    page = seq.pages[g][i]
                    if pool.hash_of(page) != h:
                        pool.publish(page, h, chunk)
                seq.hashes.append(h)
        seq.num_computed = new_len
        for g, spec in enumerate(self.groups):
            if spec.retention.keeps_everything:
                continue
            first = min(self._first_kept_page(g, new_len), len(seq.pages[g]))
            pages = seq.pages[g]
            for i in range(first):
                if pages[i] >= 0:
                    self.pools[g].release(pages[i])
                    seq.drop(g, i)

    def release(self, req) -> None:
        """Gives back everything the request holds (it ended or was preempted)."""
        seq = self.seqs.pop(req)
        for g, pages in enumerate(seq.pages):
            for p in reversed(pages):
                if p >= 0:
                    self.pools[g].release(p)
        self.slots.release(seq.state_slot)

    # ---- what a step needs ----------------------------------------------------------------------
    def block_table(self, req, group: int) -> List[int]:
        return self.seqs[req].pages[group]

    def block_table_array(self, req, group: int) -> np.ndarray:
        """The same as an int32 array (a view that the next reserve or commit may change)."""
        return self.seqs[req].table(group)

    def check_invariants(self) -> None:
        """No page lost, held twice without a count, or freed twice."""
        self.slots.check()
        held_slots = [s.state_slot for s in self.seqs.values()]
        assert len(set(held_slots)) == len(held_slots), "a state slot is held by two requests"
        for g, pool in enumerate(self.pools):
            pool.check()
            holders: Dict[int, int] = {}
            for seq in self.seqs.values():
                assert seq.table(g).tolist() == list(seq.pages[g]), "the array of a block table lags behind its list"
                for p in seq.pages[g]:
                    if p >= 0:
                        holders[p] = holders.get(p, 0) + 1
            for p in range(pool.num_pages):
                assert pool.refcount[p] == holders.get(p, 0), \
                    f"group {g} page {p}: refcount {pool.refcount[p]} but {holders.get(p, 0)} holders"
            assert pool.num_free + len(holders) == pool.num_pages
