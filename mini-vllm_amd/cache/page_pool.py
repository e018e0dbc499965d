"""Bookkeeping of the pages of one cache group: which are free, who holds them, and what
they contain (for reuse of a prompt's prefix).

Reference: minivllm/kvcache/block_manager.py. Kept from it: reference counts
(block_manager.py:76-79,100-109), the chained content hash ``xxh64(previous hash as 8 bytes LE,
then each token as 4 bytes LE signed)`` (block_manager.py:24-30), a hit only when the stored
tokens are equal too (block_manager.py:69), freed pages keeping their content until they are
handed out again (block_manager.py:80-81). Changed: the free list is first-in first-out, so
that cached content lives as long as possible (the reference pops the most recently freed id,
block_manager.py:119); the hash entry of a page is deleted when the page is handed out for new
content (the reference resets the page before it looks, block_manager.py:125-128).
"""
from __future__ import annotations

from collections import OrderedDict
from typing import Dict, List, Optional, Sequence, Tuple

try:
    import xxhash

    def _hash64(data: bytes) -> int:
        return xxhash.xxh64(data).intdigest()
except ImportError:  # pragma: no cover - xxhash is present in the supported environment
    import hashlib

    def _hash64(data: bytes) -> int:
        return int.from_bytes(hashlib.blake2b(data, digest_size=8).digest(), "little")


def page_hash(tokens: Sequence[int], prefix: Optional[int] = None) -> int:
    """Hash of one full page of tokens, chained to the hash of the page before it."""
    data = bytearray()
    if prefix is not None:
        data += int(prefix).to_bytes(8, "little")
    for t in tokens:
        data += int(t).to_bytes(4, "little", signed=True)
    return _hash64(bytes(data))


class OutOfPages(RuntimeError):
    pass


class PagePool:
    def __init__(self, num_pages: int, on_recycle=None):
        """``on_recycle(page, why)`` is told when a page is handed out for new content ("allocate")
        and when its last holder lets go of it ("release"): a debugging hook, see
        ``EngineConfig.debug_poison_pages``."""
        self.on_recycle = on_recycle
        if num_pages < 1:
            raise ValueError(f"a page pool needs at least one page, got {num_pages}")
        self.num_pages = num_pages
        self.refcount: List[int] = [0] * num_pages
        # free pages in the order they were freed (oldest first)
        self._free: "OrderedDict[int, None]" = OrderedDict((i, None) for i in range(num_pages))
        self._hash: List[Optional[int]] = [None] * num_pages
        self._tokens: List[Optional[Tuple[int, ...]]] = [None] * num_pages
        self._by_hash: Dict[int, int] = {}

    # ---- counts ---------------------------------------------------------------------------
    @property
    def num_free(self) -> int:
        return len(self._free)

    @property
    def num_used(self) -> int:
        return self.num_pages - len(self._free)

    def is_free(self, page: int) -> bool:
        return page in self._free

    # ---- handing out and taking back --------------------------------------------------------
    def allocate(self) -> int:
        """The longest-free page, for new content; what it held is forgotten."""
        if not self._free:
            raise OutOfPages("no free page")
        page, _ = self._free.popitem(last=False)
        self._forget(page)
        assert self.refcount[page] == 0
        self.refcount[page] = 1
        if self.on_recycle is not None:
            self.on_recycle(page, "allocate")
        return page

    def share(self, page: int) -> None:
        """Another holder of a page whose content is reused. A free page is revived."""
        if page in self._free:
            del self._free[page]
            assert self.refcount[page] == 0
        else:
            assert self.refcount[page] >= 1
        self.refcount[page] += 1

    def release(self, page: int) -> None:
        if self.refcount[page] <= 0:
            raise AssertionError(f"page {page} is released more often than it was taken")
        self.refcount[page] -= 1
        if self.refcount[page] == 0:
            self._free[page] = None
            if self.on_recycle is not None:
                self.on_recycle(page, "release")

    # ---- content ----------------------------------------------------------------------------
    def _forget(self, page: int) -> None:
        h = self._hash[page]
        if h is not None and self._by_hash.get(h) == page:
            del self._by_hash[h]
        self._hash[page] = None
        self._tokens[page] = None

    def publish(self, page: int, h: int, tokens: Sequence[int]) -> None:
        """Records that ``page`` is full and holds ``tokens`` (hash ``h``, chained)."""
        self._forget(page)
        self._hash[page] = h
        self._tokens[page] = tuple(tokens)
        self._by_hash.setdefault(h, page)

    def lookup(self, h: int, tokens: Sequence[int]) -> Optional[int]:
        page = self._by_hash.get(h)
        if page is None or self._tokens[page] != tuple(tokens):
            return None
        return page

    def hash_of(self, page: int) -> Optional[int]:
        return self._hash[page]

    @property
    def num_hashed(self) -> int:
        return len(self._by_hash)

    def check(self) -> None:
        for p in range(self.num_pages):
            assert self.refcount[p] >= 0
            assert (self.refcount[p] == 0) == (p in self._free), f"page {p}: refcount {self.refcount[p]} vs free list"
        for h, p in self._by_hash.items():
            assert self._hash[p] == h
