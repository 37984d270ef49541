"""The cache manager: everything a request holds between steps.

It owns the groups of pages (pages.py), the state slots (state.py), the length
of every request, and, when given an allocator, the device tensors behind them.
The host logic runs without a GPU; device work (page copies for copy-on-write,
zeroing of a fresh state slot) goes through two callbacks.

Per step the step function calls `append_many([(request, n_tokens), ...])`,
which is atomic: either every request gets its slots in every group, or
OutOfPages is raised and no request has gained a token, a slot or a page (the
reference preflights every layer before mutating any, runtime/model.py:98-102);
the only thing a refused step may have done is to give back pages that a window
had passed, which no later query reads.
"""
from dataclasses import dataclass, field

from .pages import CacheGroup, OutOfPages
from .state import StateSlots


@dataclass
class Appended:
    """What one request got in a step."""
    request: object
    start: int                                  # position of its first new token
    count: int
    slots: dict = field(default_factory=dict)   # group id -> [count] physical token slots
    state_slot: int = 0


class CacheManager:
    fast_decode = True   # steps of one token a request take a short path (tests switch it off to compare)

    def __init__(self, site_needs, n_pages, page_size, max_requests, state_needs=None,
                 allocate_pages=None, allocate_state=None, copy_pages=None, zero_state=None, copy_state=None):
        """site_needs: {site id: need (KVNeed or another class with its methods)}; state_needs: {site id: StateNeed}.
        n_pages: pages per group (an int, or {need: int}).  `allocate_pages(shape)` makes a group's device storage,
        of the shape its need states."""
        self.page_size = page_size
        self.groups = []
        self.group_of_site = {}
        by_need = {}
        for site, need in site_needs.items():
            by_need.setdefault(need, []).append(site)
        for gid, (need, sites) in enumerate(by_need.items()):
            pages = n_pages[need] if isinstance(n_pages, dict) else n_pages
            group = CacheGroup(need, sites, pages, page_size)
            if allocate_pages is not None:
                group.storage = allocate_pages(need.storage_shape(len(sites), pages, page_size))
            self.groups.append(group)
            for index, site in enumerate(sites):
                self.group_of_site[site] = (gid, index)
        self.lengths = {}
        self.slots = StateSlots(max_requests)
        self.state_needs = dict(state_needs or {})
        self.state_storage = {}
        if allocate_state is not None:
            for site, need in self.state_needs.items():
                self.state_storage[site] = allocate_state(max_requests, need.shape, need.dtype)
        self._copy_pages, self._zero_state, self._copy_state = copy_pages, zero_state, copy_state

    # -- requests ---------------------------------------------------------
    def create(self, request):
        if request in self.lengths:
            raise ValueError(f"duplicate request {request!r}")
        slot = self.slots.acquire(request)
        self.lengths[request] = 0
        for group in self.groups:
            group.create(request)
        if self._zero_state is not None:
            for site in self.state_needs:
                self._zero_state(self.state_storage[site], slot)
        return slot

    def fork(self, source, target):
        """target starts as a copy of source: pages shared, state copied."""
        if target in self.lengths:
            raise ValueError(f"duplicate request {target!r}")
        slot = self.slots.acquire(target)
        self.lengths[target] = self.lengths[source]
        for group in self.groups:
            group.fork(source, target)
        if self._copy_state is not None:
            for site in self.state_needs:
                self._copy_state(self.state_storage[site], self.slots.slot_of(source), slot)
        return slot

    def release(self, request):
        """Give back everything the request holds.  The caller makes sure no
        device work that reads its pages is still running."""
        del self.lengths[request]
        for group in self.groups:
            group.release(request)
        self.slots.release(request)

    def __contains__(self, request):
        return request in self.lengths

    def length(self, request):
        return self.lengths[request]

    # -- appending ----------------------------------------------------------
    def pages_needed(self, items):
        """Per group: fresh pages minus pages a window gives back first."""
        out = []
        for group in self.groups:
            need = 0
            for request, n in items:
                length = self.lengths[request]
                need += group.pages_needed(request, length, n) - group.trimmable(request, length)
            out.append(need)
        return out

    def can_append(self, items):
        return all(need <= len(group.pool.free) for need, group in zip(self.pages_needed(items), self.groups))

    def append_many(self, items, commit=True):
        """items: [(request, n_new)], each request at most once.  Returns [Appended].
        With commit=False the slots are placed but the requests' lengths stay: the caller calls `commit(done)`
        once the step that writes the slots is launched, or `abandon(done)` if it could not be."""
        seen = set()
        for request, n in items:
            if request not in self.lengths:
                raise KeyError(f"unknown request {request!r}")
            if request in seen:
                raise ValueError(f"request {request!r} appears twice in one step")
            if n <= 0:
                raise ValueError("a request must bring at least one token")
            seen.add(request)
        if self.fast_decode and all(n == 1 for _, n in items) and all(g.need.window is None for g in self.groups):
            return self._append_one_each(items, commit)
        # Windows first give back, for every request of the step, the pages that no later query can see; only then
        # are fresh pages counted and taken.  (Trimmed one request at a time, a request that needs a page could
        # come before the one whose window frees it, and run out in the middle of the step.)  Giving such a page
        # back changes nothing that a retry of the step would read.
        for request, _ in items:
            for group in self.groups:
                group.trim(request, self.lengths[request])
        if not self.can_append(items):
            raise OutOfPages("not enough free KV pages for this step")
        result = []
        for request, n in items:
            length = self.lengths[request]
            done = Appended(request, length, n, state_slot=self.slots.slot_of(request))
            for gid, group in enumerate(self.groups):
                slots, copies = group.append(request, length, n)
                done.slots[gid] = slots
                if copies and self._copy_pages is not None:
                    self._copy_pages(group, copies)
            if commit:
                self.lengths[request] = length + n
            result.append(done)
        return result

    def commit(self, done):
        """The step that fills the slots of `done` (append_many with commit=False) is on its way: the tokens count.
        (On its way, not finished: later steps read the slots only because they are queued on the same stream.)"""
        for d in done:
            if self.lengths[d.request] != d.start:
                raise RuntimeError(f"request {d.request!r} moved between its append and its commit")
            self.lengths[d.request] = d.start + d.count
        return done

    def abandon(self, done):
        """The step of `done` (append_many with commit=False) was never launched, or failed on its way: pages taken
        for its tokens go back, the requests' lengths and tables stand where they stood.  (A page copied for a write
        stays copied, pages that a window had passed stay given back: neither changes what a later step reads.)
        Kernels of the failed step may still be queued and write into pages that go back here, and the page copy of
        a copy-on-write may still be on its way: whoever takes those pages next must be ordered behind them.  The
        owner launches everything on ONE stream (ModelRunner refuses a step on another), which is that order.
        Per-request state is not restored: see ModelRunner.step."""
        for d in done:
            keep = -(-self.lengths[d.request] // self.page_size)
            for group in self.groups:
                table = group.tables[d.request]
                while len(table) > keep:
                    group.pool.drop(table.pop())
                    group._touch(d.request)

    def _append_one_each(self, items, commit=True):
        """append_many for the common step in which every request brings one token and no group has a
        window: the same pages in the same order, with the counting and the placing done in line."""
        P = self.page_size
        lengths = self.lengths
        for group in self.groups:
            refs, tables, fresh = group.pool.refs, group.tables, 0
            for request, _ in items:
                if lengths[request] % P == 0 or refs[tables[request][-1]] > 1:
                    fresh += 1
            if fresh > len(group.pool.free):
                raise OutOfPages("not enough free KV pages for this step")
        result = []
        for request, _ in items:
            length = lengths[request]
            done = Appended(request, length, 1, state_slot=self.slots.slot_of(request))
            for gid, group in enumerate(self.groups):
                table = group.tables[request]
                if length % P == 0:
                    table.append(group.pool.allocate())
                    group._touch(request)
                elif group.pool.refs[table[-1]] > 1:      # the shared, partly filled last page: copy on write
                    slots, copies = group.append(request, length, 1)
                    if copies and self._copy_pages is not None:
                        self._copy_pages(group, copies)
                done.slots[gid] = [table[-1] * P + length % P]
            if commit:
                lengths[request] = length + 1
            result.append(done)
        return result

    def trim(self, request):
        """Give back pages that a window has passed (also done by every append)."""
        for group in self.groups:
            group.trim(request, self.lengths[request])

    def table(self, gid, request):
        return self.groups[gid].tables[request]

    # -- views for mixers ---------------------------------------------------
    def pages_of_site(self, site):
        """(group id, *views): the group a site's pages belong to and the site's own views of the group's storage,
        as its need lays them out (KVNeed: keys [pages, kv_heads, P, D], values [pages, kv_heads, D, P])."""
        gid, index = self.group_of_site[site]
        group = self.groups[gid]
        return (gid, *group.need.views(group.storage, index))

    kv_of_site = pages_of_site

    # -- bookkeeping --------------------------------------------------------
    def check(self):
        for group in self.groups:
            group.check()
            assert set(group.tables) == set(self.lengths), "a group knows other requests than the manager"
            for request, table in group.tables.items():
                assert len(table) == -(-self.lengths[request] // group.page_size), "table length differs from token count"
        self.slots.check()
        assert set(self.slots.owner) == set(self.lengths)

    def free_pages(self):
        return [len(g.pool.free) for g in self.groups]

    def capacity(self):
        """Pages of each group's pool."""
        return [g.pool.n_pages for g in self.groups]

    def most_pages_held(self, tokens, portion):
        """Per group, the most pages one request holds at any time while it grows to `tokens` cached tokens in
        steps of at most `portion`: all of them where every key is kept; where only a window is kept, the pages
        that a window and a portion can touch (a portion is placed after the pages behind its first token's
        window went back)."""
        P = self.page_size
        out = []
        for group in self.groups:
            pages = -(-tokens // P)
            if group.need.window is not None:
                pages = min(pages, (group.need.window + max(1, portion) - 1) // P + 2)
            out.append(pages)
        return out

    def report(self):
        out = []
        for gid, g in enumerate(self.groups):
            token_bytes = g.need.elements_per_token() * len(g.sites)
            out.append({"group": gid, "sites": len(g.sites), "window": g.need.window, "pages": g.pool.n_pages,
                        "resident_pages": g.pool.used, "peak_pages": g.pool.peak, "free_pages": len(g.pool.free),
                        "shared_pages": sum(1 for r in g.pool.refs if r > 1), "requests": len(g.tables),
                        "elements_per_token": token_bytes})
        return out


def pages_that_fit(site_needs, page_size, itemsize, free_bytes, fraction=0.8, most=None):
    """How many pages a pool may have so that the caches of all sites take `fraction` of `free_bytes`:
    a page index costs, in every site that keeps pages, page_size times the elements its need takes a token.
    `most` caps the answer (more pages than the requests can ever address are of no use)."""
    per_page = sum(need.elements_per_token() * page_size * itemsize for need in site_needs.values() if need is not None)
    if per_page == 0:
        return 1
    pages = int(free_bytes * fraction) // per_page
    if most is not None:
        pages = min(pages, most)
    if pages < 1:
        raise MemoryError(f"no room for a single cache page ({per_page} bytes) in {free_bytes} free bytes")
    return pages

