"""Host bookkeeping of one pool of pages: who holds a page, which pages are
free, and which free or held pages carry known content.

The pool hands out page ids only; the device memory behind an id belongs to
the cache group.  A page is either held (ref count > 0) or on the free list,
ordered from least to most recently released; `alloc` takes the oldest.  A
full page can be sealed: its tokens and the hash chained from the pages before
it go into a content index, so that a later request with the same beginning
adopts the page instead of computing it again; a sealed page that became free
stays in the index until it is taken for new content
(/root/reference/src/kipp_kv_pool.c:13-22, 202-269).
"""
from __future__ import annotations

import math
from collections import OrderedDict
from dataclasses import dataclass
from typing import Dict, List, Optional, Sequence, Tuple

_FNV_OFFSET = 1469598103934665603
_FNV_PRIME = 1099511628211
_MASK = (1 << 64) - 1


def chain_hash(parent: int, tokens: Sequence[int]) -> int:
    """FNV-1a over the parent hash's 8 bytes, then each token's 4 bytes, low byte
    first (/root/reference/src/kipp_kv_pool.c:48-64)."""
    h = _FNV_OFFSET
    for shift in range(0, 64, 8):
        h = ((h ^ ((parent >> shift) & 0xFF)) * _FNV_PRIME) & _MASK
    for tok in tokens:
        for shift in range(0, 32, 8):
            h = ((h ^ ((tok >> shift) & 0xFF)) * _FNV_PRIME) & _MASK
    return h


@dataclass
class PoolStats:
    total_pages: int
    free_pages: int
    reused_pages_total: int
    evicted_pages_total: int


def scattered_order(n: int) -> List[int]:
    """0 .. n-1 in an order in which neighbours lie far apart (steps of about 0.618 n, coprime
    to n).  A fresh pool hands its pages out in this order: sequences that arrive together and
    have the same length would otherwise lie at equal distances in memory, a power of two for
    prompts of 2,048 tokens, and kernels that walk all of them in step would find every sequence's
    current page in the same memory channel (measured: decode attention of 128 such sequences a
    fifth slower)."""
    step = max(1, int(n * 0.6180339887))
    while math.gcd(step, n) != 1:
        step += 1
    return [(i * step) % n for i in range(n)]


class PagePool:
    def __init__(self, num_pages: int, page_size: int, order: Optional[Sequence[int]] = None):
        """`order`: the order in which a fresh pool hands its pages out (a permutation of
        0 .. num_pages - 1; default `scattered_order`).  Where a request's pages lie must not change
        its results; tests run one trace under several orders."""
        if num_pages <= 0 or page_size <= 0:
            raise ValueError("a pool needs at least one page of at least one token")
        order = scattered_order(num_pages) if order is None else [int(p) for p in order]
        if sorted(order) != list(range(num_pages)):
            raise ValueError("the order of a pool's pages must name every page once")
        self.num_pages = num_pages
        self.page_size = page_size
        self.ref = [0] * num_pages
        self.free: "OrderedDict[int, None]" = OrderedDict((i, None) for i in order)
        self.content: List[Optional[Tuple[int, Tuple[int, ...]]]] = [None] * num_pages  # (hash, tokens) if indexed
        self.index: Dict[int, List[int]] = {}
        self.reused_total = 0
        self.evicted_total = 0
        self.force_hash: Optional[int] = None  # tests: make every hash collide

    # -- hashing ---------------------------------------------------------------
    def _hash(self, parent: int, tokens: Sequence[int]) -> int:
        return self.force_hash if self.force_hash is not None else chain_hash(parent, tokens)

    # -- allocation ------------------------------------------------------------
    @property
    def free_count(self) -> int:
        return len(self.free)

    def _drop_from_index(self, page: int) -> None:
        entry = self.content[page]
        if entry is None:
            return
        chain = self.index.get(entry[0], [])
        if page in chain:
            chain.remove(page)
            if not chain:
                del self.index[entry[0]]
        self.content[page] = None

    def alloc(self) -> Optional[int]:
        """The least recently released free page as a private page (ref 1), or None."""
        if not self.free:
            return None
        page, _ = self.free.popitem(last=False)
        if self.content[page] is not None:
            self._drop_from_index(page)
            self.evicted_total += 1
        self.ref[page] = 1
        return page

    def retain(self, page: int) -> None:
        if self.ref[page] == 0:
            del self.free[page]
        self.ref[page] += 1

    def release(self, page: int) -> None:
        """Give one hold back; at zero the page becomes free (and stays indexed).
        Releasing a free page is an error of the caller and raises."""
        if not 0 <= page < self.num_pages or self.ref[page] <= 0:
            raise ValueError(f"page {page} is released but not held")
        self.ref[page] -= 1
        if self.ref[page] == 0:
            self.free[page] = None

    # -- content ---------------------------------------------------------------
    def _lookup(self, h: int, tokens: Tuple[int, ...]) -> Optional[int]:
        for page in self.index.get(h, ()):
            entry = self.content[page]
            if entry is not None and entry[1] == tokens:  # verify by tokens, never by hash alone
                return page
        return None

    def seal(self, page: int, parent: int, tokens: Sequence[int]) -> int:
        """Publish a full held page; returns its hash.  If the same content is
        already indexed the page stays private."""
        tokens = tuple(int(t) for t in tokens)
        if len(tokens) != self.page_size:
            raise ValueError("only full pages are sealed")
        if self.ref[page] <= 0:
            raise ValueError(f"page {page} is sealed but not held")
        if self.content[page] is not None:
            raise ValueError(f"page {page} is sealed twice")
        h = self._hash(parent, tokens)
        if self._lookup(h, tokens) is None:
            self.content[page] = (h, tokens)
            self.index.setdefault(h, []).append(page)
        return h

    def prefix_match(self, tokens: Sequence[int]) -> Tuple[List[int], int]:
        """Pages holding the longest known beginning of `tokens`, each retained
        for the caller, and the chained hash after them.  At most
        (len - 1) // page_size pages, so one token is always left to run
        (/root/reference/src/kipp_kv_pool.c:271-304)."""
        limit = (len(tokens) - 1) // self.page_size if tokens else 0
        pages: List[int] = []
        parent = 0
        for i in range(limit):
            chunk = tuple(int(t) for t in tokens[i * self.page_size:(i + 1) * self.page_size])
            h = self._hash(parent, chunk)
            page = self._lookup(h, chunk)
            if page is None:
                break
            self.retain(page)
            self.reused_total += 1
            pages.append(page)
            parent = h
        return pages, parent

    # -- inspection ------------------------------------------------------------
    def stats(self) -> PoolStats:
        return PoolStats(self.num_pages, len(self.free), self.reused_total, self.evicted_total)

    def check(self) -> None:
        """Invariants: every page is either held or free, never both; indexed
        pages are where the index says."""
        for page in range(self.num_pages):
            held, free = self.ref[page] > 0, page in self.free
            if held == free:
                raise AssertionError(f"page {page}: ref {self.ref[page]}, on free list: {free}")
            if self.ref[page] < 0:
                raise AssertionError(f"page {page}: negative ref count")
        for h, chain in self.index.items():
            for page in chain:
                if self.content[page] is None or self.content[page][0] != h:
                    raise AssertionError(f"index entry of page {page} is stale")
