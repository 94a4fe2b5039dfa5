"""Which pages of one pool are free, in use, or free but still holding a reusable prefix
(behaviour of reference atomserve/block_allocator.py:33-129).

A page is in exactly one state: in use (reference count > 0), free and cached (count
0, still named by a content hash, revivable through `lookup`/`acquire`), or free and
empty.  Both free states wait in one queue, oldest first; `allocate` takes from its
head, and taking a cached page forgets its hash.  The queue is an intrusive doubly
linked list over page ids, so reviving a page from its middle is O(1).

Pure bookkeeping over integers: no tensors, usable without a GPU.
"""

import hashlib
import struct

_NIL = -1


def blocks_for_tokens(num_tokens: int, block_size: int) -> int:
    """Pages needed to hold `num_tokens` tokens."""
    return (num_tokens + block_size - 1) // block_size


def page_hash(parent: bytes, tokens) -> bytes:
    """Content address of a full page: its tokens chained onto the hash of the page before it
    (b"" for the first), so equal hashes mean equal prefixes
    (reference atomserve/block_allocator.py:38-46)."""
    return hashlib.sha256(parent + struct.pack(f"<{len(tokens)}I", *tokens)).digest()


class OutOfPagesError(RuntimeError):
    """More pages were asked for than are free."""


class PageAllocator:
    def __init__(self, num_pages: int):
        if num_pages < 1:
            raise ValueError("a pool needs at least one page")
        self.num_pages = num_pages
        self._refs = [0] * num_pages
        # free queue: head is the oldest; every page starts free, in id order
        self._next = [i + 1 for i in range(num_pages)]
        self._next[-1] = _NIL
        self._prev = [i - 1 for i in range(num_pages)]
        self._head, self._tail = 0, num_pages - 1
        self._queued = [True] * num_pages
        self._num_free = num_pages
        self._hash_of_page: dict = {}
        self._page_of_hash: dict = {}

    # ---- the free queue -------------------------------------------------------------
    def _unlink(self, page: int) -> None:
        p, n = self._prev[page], self._next[page]
        if p == _NIL:
            self._head = n
        else:
            self._next[p] = n
        if n == _NIL:
            self._tail = p
        else:
            self._prev[n] = p
        self._queued[page] = False
        self._num_free -= 1

    def _append(self, page: int) -> None:
        self._prev[page], self._next[page] = self._tail, _NIL
        if self._tail == _NIL:
            self._head = page
        else:
            self._next[self._tail] = page
        self._tail = page
        self._queued[page] = True
        self._num_free += 1

    # ---- counts -----------------------------------------------------------------------
    @property
    def num_free(self) -> int:
        """Pages that `allocate` could hand out now (cached ones are evicted on demand)."""
        return self._num_free

    @property
    def num_cached(self) -> int:
        """Pages named by a prefix hash, in use or not."""
        return len(self._page_of_hash)

    def refcount(self, page: int) -> int:
        return self._refs[page]

    # ---- pages ------------------------------------------------------------------------
    def allocate(self, n: int) -> list:
        """Take `n` free pages, oldest first; all or nothing."""
        if n > self._num_free:
            raise OutOfPagesError(f"need {n} KV blocks, only {self._num_free} free")
        taken = []
        for _ in range(n):
            page = self._head
            self._unlink(page)
            stale = self._hash_of_page.pop(page, None)
            if stale is not None:  # about to be overwritten: its hash must not find it any more
                del self._page_of_hash[stale]
            self._refs[page] = 1
            taken.append(page)
        return taken

    def free(self, pages) -> None:
        """Drop one reference to each page.  Given in a request's order, they are released
        last page first, so that the head of a shared prefix is evicted last."""
        pages = list(pages)
        for page in pages:
            if not 0 <= page < self.num_pages or self._refs[page] == 0:
                raise ValueError(f"block {page} is not allocated")
        counts: dict = {}
        for page in pages:
            counts[page] = counts.get(page, 0) + 1
            if counts[page] > self._refs[page]:
                raise ValueError(f"block {page} is not allocated")
        for page in reversed(pages):
            self._refs[page] -= 1
            if self._refs[page] == 0:
                self._append(page)

    # ---- prefix cache -----------------------------------------------------------------
    def lookup(self, h: bytes):
        """The page holding the prefix with hash `h`, if one still does."""
        return self._page_of_hash.get(h)

    def acquire(self, page: int) -> None:
        """Add a reference to a page found by `lookup`, taking it out of the free queue if there."""
        if self._refs[page] == 0:
            if not self._queued[page]:
                raise ValueError(f"block {page} is neither in use nor free")
            self._unlink(page)
        self._refs[page] += 1

    def register(self, page: int, h: bytes) -> None:
        """Name a full, computed page by its prefix hash; the first page to hold a prefix stays
        its cached copy."""
        if h not in self._page_of_hash and page not in self._hash_of_page:
            self._page_of_hash[h] = page
            self._hash_of_page[page] = h

    def check(self) -> None:
        """Internal consistency: every page is either referenced or queued, never both."""
        seen, page, count = set(), self._head, 0
        while page != _NIL:
            assert page not in seen and self._refs[page] == 0 and self._queued[page]
            seen.add(page)
            count += 1
            page = self._next[page]
        assert count == self._num_free
        for page in range(self.num_pages):
            assert (self._refs[page] == 0) == (page in seen), page
        for h, page in self._page_of_hash.items():
            assert self._hash_of_page[page] == h
