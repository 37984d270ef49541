"""Host-side ownership of cache pages: one pool and one set of block tables per
group of layers with the same need.

A *need* says what a mixer keeps per token: keys and values of a given shape,
either all of them or only a trailing window.  Layers (cache sites) with equal
needs form a group; a group has pages of its own, and one page index is valid in
every site of its group.  Each request has one block table per group: entry j
is the physical page of logical tokens j*P..j*P+P-1, or -1 once a window has
passed that page and it was given back.

Ownership follows the reference's PagedCache (runtime/cache.py:9-118): a free
stack popped from the low end first, a reference count per page, fork by
sharing, copy-on-write of a shared, partly filled last page, exhaustion that
changes nothing.  Unlike it, there is one table per request per group (not one
per layer) and an append may bring many tokens.
"""
from dataclasses import dataclass
from typing import Optional

import numpy as np


class OutOfPages(MemoryError):
    pass


@dataclass(frozen=True)
class KVNeed:
    """Keys and values per token: [kv_heads, head_dim] each; window None = all keys.

    A need is what the cache manager knows of a mixer's pages.  The manager groups sites by equal needs and asks the
    need, never itself, how the pages of a group are stored: any frozen dataclass with `window` and the four
    methods below can stand here (keys and values of different widths, a compressed form, one tensor a token).
    This one's layout is what the attention kernels of this package read: a page's keys as [kv_heads, page_size,
    head_dim], its values transposed as [kv_heads, head_dim, page_size], keys of all pages first."""
    kv_heads: int
    head_dim: int
    window: Optional[int] = None

    def elements_per_token(self):
        """Cached elements a token takes in one site."""
        return 2 * self.kv_heads * self.head_dim

    def storage_shape(self, sites, pages, page_size):
        """Shape of the one tensor that holds the pages of `sites` sites of a group."""
        return (sites, 2, pages, self.kv_heads, page_size, self.head_dim)

    def slabs(self, sites):
        """Into how many contiguous runs of `pages` pages the storage divides (a page copy touches each)."""
        return sites * 2

    def views(self, storage, index):
        """What a mixer reads and writes of site `index` of the group: (keys [pages, kv_heads, P, D],
        values [pages, kv_heads, D, P])."""
        pages, kv_heads, psize, dim = storage.shape[2:]
        return storage[index, 0], storage[index, 1].view(pages, kv_heads, dim, psize)


@dataclass(frozen=True)
class StateNeed:
    """A fixed-size state per request."""
    shape: tuple
    dtype: str = "float32"


class PagePool:
    def __init__(self, n_pages):
        if n_pages <= 0:
            raise ValueError("a page pool needs at least one page")
        self.n_pages = n_pages
        self.refs = [0] * n_pages
        self.free = list(reversed(range(n_pages)))  # page 0 is handed out first
        self.peak = 0

    def allocate(self):
        if not self.free:
            raise OutOfPages("KV page pool exhausted")
        page = self.free.pop()
        self.refs[page] = 1
        self.peak = max(self.peak, self.n_pages - len(self.free))
        return page

    def share(self, page):
        if self.refs[page] <= 0:
            raise AssertionError(f"page {page} is shared while free")
        self.refs[page] += 1

    def drop(self, page):
        if self.refs[page] <= 0:
            raise AssertionError(f"page {page} is freed twice")
        self.refs[page] -= 1
        if self.refs[page] == 0:
            self.free.append(page)

    @property
    def used(self):
        return self.n_pages - len(self.free)


class CacheGroup:
    """Pages and block tables of the sites that share one KVNeed."""

    def __init__(self, need, sites, n_pages, page_size):
        if page_size <= 0:
            raise ValueError("page size must be positive")
        self.need, self.sites = need, list(sites)
        self.page_size = page_size
        self.pool = PagePool(n_pages)
        self.tables = {}
        self.versions = {}   # request -> stamp of the last change of its table (stamps are never reused)
        self._stamp = 0
        self.storage = None  # device tensor of the shape the need states (storage_shape), set by the owner

    # -- planning -------------------------------------------------------
    def _dead_pages(self, request, length):
        """Logical pages that no later query can see (window groups only)."""
        if self.need.window is None:
            return 0
        first_visible = max(0, length - self.need.window + 1)  # the next token sits at `length`
        return first_visible // self.page_size

    def pages_needed(self, request, length, n_new):
        """Fresh pages an append of n_new tokens takes (after trimming)."""
        table = self.tables[request]
        have = len(table)
        want = -(-(length + n_new) // self.page_size)
        need = max(0, want - have)
        if n_new > 0 and length % self.page_size and table[-1] >= 0 and self.pool.refs[table[-1]] > 1:
            need += 1  # copy-on-write of the shared, partly filled last page
        return need

    def trimmable(self, request, length):
        table = self.tables[request]
        return sum(1 for j in range(min(self._dead_pages(request, length), len(table)))
                   if table[j] >= 0 and self.pool.refs[table[j]] == 1)

    # -- mutation -------------------------------------------------------
    def _touch(self, request):
        self._stamp += 1
        self.versions[request] = self._stamp

    def trim(self, request, length):
        table = self.tables[request]
        for j in range(min(self._dead_pages(request, length), len(table))):
            if table[j] >= 0:
                self.pool.drop(table[j])
                table[j] = -1
                self._touch(request)

    def append(self, request, length, n_new):
        """Slots of the n_new tokens at logical positions length.. and the page
        copies (src, dst) that must run on the device before they are written."""
        table, P = self.tables[request], self.page_size
        copies = []
        if n_new > 0 and length % P and self.pool.refs[table[-1]] > 1:
            old, new = table[-1], self.pool.allocate()
            copies.append((old, new))
            self.pool.drop(old)
            table[-1] = new
            self._touch(request)
        while len(table) * P < length + n_new:
            table.append(self.pool.allocate())
            self._touch(request)
        if n_new > 32:      # a prompt portion: the same, vectorised
            at = np.arange(length, length + n_new, dtype=np.int64)
            slots = (np.asarray(table, dtype=np.int64)[at // P] * P + at % P).tolist()
        else:
            slots = [table[(length + i) // P] * P + (length + i) % P for i in range(n_new)]
        return slots, copies

    def create(self, request):
        self.tables[request] = []
        self._touch(request)

    def fork(self, source, target):
        self.tables[target] = list(self.tables[source])
        self._touch(target)
        for page in self.tables[target]:
            if page >= 0:
                self.pool.share(page)

    def release(self, request):
        self.versions.pop(request, None)
        for page in self.tables.pop(request):
            if page >= 0:
                self.pool.drop(page)

    def check(self):
        expected = [0] * self.pool.n_pages
        for table in self.tables.values():
            for page in table:
                if page >= 0:
                    expected[page] += 1
        assert expected == self.pool.refs, "reference counts differ from table occurrences"
        free = self.pool.free
        assert len(free) == len(set(free)), "a page is on the free list twice"
        assert set(free) == {p for p, r in enumerate(self.pool.refs) if r == 0}, "free list differs from unreferenced pages"
