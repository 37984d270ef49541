"""The cache manager on the host: no page lost, held twice or freed twice, under
random orders of requests; copy-on-write; windows giving pages back; state slots."""
import random

import pytest

from runtime.cache import CacheManager, KVNeed, OutOfPages, StateNeed, StateSlots


def manager(pages=8, page_size=4, sites=2, window=None, max_requests=8, **kw):
    needs = {i: KVNeed(2, 16, None) for i in range(sites)}
    if window:
        needs[sites] = KVNeed(2, 16, window)
    return CacheManager(needs, pages, page_size, max_requests, **kw)


def test_append_slots_follow_the_block_table():
    m = manager()
    m.create("a")
    (d,) = m.append_many([("a", 6)])
    assert d.start == 0 and d.count == 6 and m.length("a") == 6
    table = m.table(0, "a")
    assert len(table) == 2
    assert d.slots[0] == [table[i // 4] * 4 + i % 4 for i in range(6)]
    (d,) = m.append_many([("a", 3)])
    assert d.start == 6 and d.slots[0][:2] == [table[1] * 4 + 2, table[1] * 4 + 3] and len(m.table(0, "a")) == 3
    m.check()


def test_report_counts_resident_peak_free_and_shared_pages():
    # reference runtime/cache.py:109-118 (pool, resident, peak, free, shared, sequences)
    m = manager(pages=8, page_size=4, sites=2)
    m.create("a")
    m.append_many([("a", 9)])                      # three pages
    m.fork("a", "b")                               # shared by two requests
    m.append_many([("b", 1)])                      # copy-on-write of the partly filled last page
    (r,) = m.report()
    assert r["sites"] == 2 and r["pages"] == 8 and r["requests"] == 2 and r["window"] is None
    assert r["resident_pages"] == 4 and r["free_pages"] == 4 and r["shared_pages"] == 2 and r["peak_pages"] == 4
    assert r["elements_per_token"] == 2 * 2 * 16 * 2
    m.release("a"); m.release("b")
    (r,) = m.report()
    assert r["resident_pages"] == 0 and r["free_pages"] == 8 and r["peak_pages"] == 4 and r["requests"] == 0
    m.check()


def test_sites_with_equal_needs_share_one_group():
    m = manager(sites=3, window=5)
    assert len(m.groups) == 2 and len(m.groups[0].sites) == 3 and m.groups[1].need.window == 5
    assert m.group_of_site[2] == (0, 2) and m.group_of_site[3] == (1, 0)


def test_exhaustion_is_atomic_and_duplicates_are_rejected():
    # reference tests/test_cache.py:20-31 and tests/test_model.py:42-46
    m = manager(pages=2, page_size=2)
    m.create("a"); m.create("b")
    with pytest.raises(ValueError):
        m.create("a")
    m.append_many([("a", 3)])
    before = (m.length("a"), m.length("b"), list(m.table(0, "a")), m.free_pages())
    with pytest.raises(OutOfPages):
        m.append_many([("a", 1), ("b", 1)])   # a fits in its page, b needs a third page
    assert before == (m.length("a"), m.length("b"), list(m.table(0, "a")), m.free_pages())
    m.check()
    with pytest.raises(ValueError):
        m.append_many([("a", 1), ("a", 1)])
    with pytest.raises(KeyError):
        m.append_many([("zzz", 1)])


def test_fork_shares_pages_and_copies_a_partial_page_on_write():
    # reference tests/test_cache.py:7-18
    copies = []
    m = manager(pages=3, page_size=2, sites=1, copy_pages=lambda g, c: copies.extend(c))
    m.create("a")
    m.append_many([("a", 1)])
    m.fork("a", "b")
    assert m.table(0, "a") == m.table(0, "b") and m.groups[0].pool.refs[m.table(0, "a")[0]] == 2
    (d,) = m.append_many([("b", 1)])
    assert m.table(0, "a") != m.table(0, "b") and m.length("a") == 1 and m.length("b") == 2
    assert copies == [(m.table(0, "a")[0], m.table(0, "b")[0])]
    assert d.slots[0] == [m.table(0, "b")[0] * 2 + 1]
    m.check()
    m.release("a"); m.release("b"); m.check()
    assert m.free_pages() == [3]


def test_fork_at_a_page_edge_copies_nothing():
    copies = []
    m = manager(pages=4, page_size=2, sites=1, copy_pages=lambda g, c: copies.extend(c))
    m.create("a"); m.append_many([("a", 2)]); m.fork("a", "b")
    m.append_many([("b", 3)]); m.append_many([("a", 1)])
    assert not copies and m.table(0, "a")[0] == m.table(0, "b")[0] and m.table(0, "a")[1] != m.table(0, "b")[1]
    m.check()


def test_pages_are_reused_lowest_first_after_release():
    m = manager(pages=4, page_size=2, sites=1)
    m.create("a"); m.append_many([("a", 8)])
    with pytest.raises(OutOfPages):
        m.create("b"); m.append_many([("b", 1)])
    m.release("a")
    assert m.free_pages() == [4]
    m.append_many([("b", 5)])
    assert sorted(m.table(0, "b")) == sorted(set(m.table(0, "b"))) and len(m.table(0, "b")) == 3
    m.check()


def test_window_gives_pages_back_once_passed():
    m = manager(pages=6, page_size=4, sites=1, window=6)
    m.create("a")
    full, win = 0, 1
    m.append_many([("a", 4)])
    for _ in range(16):
        m.append_many([("a", 1)])
        m.check()
    # length 20: the next query (position 20) sees keys 15..20, i.e. logical pages 3.. -> pages 0,1,2 are back
    assert m.table(win, "a")[:3] == [-1, -1, -1] and all(p >= 0 for p in m.table(win, "a")[3:])
    assert all(p >= 0 for p in m.table(full, "a"))
    assert m.groups[win].pool.used == 2 and m.groups[full].pool.used == 5
    # a long portion: pages behind the window of its FIRST token are given back before it is placed
    m.release("a"); m.create("b")
    m.append_many([("b", 9)])
    assert m.table(win, "b") .count(-1) == 0       # nothing passed yet when the portion started
    m.append_many([("b", 2)])
    assert m.table(win, "b")[0] == -1 and m.table(win, "b")[1] >= 0  # first visible key is 9-6+1 = 4: page 0 is passed
    m.check()


def test_window_step_is_atomic_whatever_the_order_of_its_requests():
    """No free page, one request of the step needs a page and a LATER one frees one through its window: the step
    is served (pages are given back for all requests before any is taken).  And when it cannot be served, no
    request has moved."""
    def fill(order):
        m = manager(pages=4, page_size=4, sites=0, window=4)
        for r in "abc":
            m.create(r)
        m.append_many([("a", 4)])              # a: one full page, its next token needs a fresh one
        m.append_many([("b", 7)])              # b: two pages; its next token (position 7) sees 4..7: page 0 is dead
        m.append_many([("c", 2)])              # c: one page, partly filled
        assert m.free_pages() == [0]
        return m, [(r, 1) for r in order]
    for order in ("cab", "abc", "bca"):
        m, items = fill(order)
        assert m.can_append(items)
        done = {d.request: d for d in m.append_many(items)}
        assert (m.length("a"), m.length("b"), m.length("c")) == (5, 8, 3)
        assert m.table(0, "b")[0] == -1 and done["a"].slots[0][0] % 4 == 0
        m.check()
    # without b in the step nothing is freed: the step is refused and nobody has moved
    m, _ = fill("ca")
    before = ({r: m.length(r) for r in "abc"}, {r: list(m.table(0, r)) for r in "abc"})
    with pytest.raises(OutOfPages):
        m.append_many([("c", 1), ("a", 1)])
    assert before == ({r: m.length(r) for r in "abc"}, {r: list(m.table(0, r)) for r in "abc"})
    m.check()


@pytest.mark.parametrize("fast", [True, False])
def test_slots_without_commit_can_be_abandoned_or_committed(fast):
    """A step places its slots first and counts its tokens only once it is launched; a step that is never
    launched gives its pages back and leaves every request where it stood."""
    m = manager(pages=6, page_size=4, sites=1)
    m.fast_decode = fast
    m.create("a"); m.create("b")
    m.append_many([("a", 4), ("b", 3)])
    before = ({r: m.length(r) for r in "ab"}, {r: list(m.table(0, r)) for r in "ab"}, m.free_pages())
    for items in ([("a", 1), ("b", 1)], [("a", 9), ("b", 2)]):
        done = m.append_many(items, commit=False)
        assert (m.length("a"), m.length("b")) == (4, 3)          # not counted yet
        assert [d.start for d in done] == [4, 3]
        m.abandon(done)
        assert before == ({r: m.length(r) for r in "ab"}, {r: list(m.table(0, r)) for r in "ab"}, m.free_pages())
        m.check()
    done = m.append_many([("a", 1), ("b", 1)], commit=False)
    m.commit(done)
    assert (m.length("a"), m.length("b")) == (5, 4) and len(m.table(0, "a")) == 2
    m.check()
    with pytest.raises(RuntimeError):
        m.commit(done)                                            # the same step twice


def test_window_group_never_needs_more_than_window_plus_portion():
    m = manager(pages=4, page_size=4, sites=0, window=8)
    m.create("a")
    for _ in range(50):            # 200 tokens through 4 pages of 4
        m.append_many([("a", 4)])
        m.check()
    assert m.length("a") == 200 and m.groups[0].pool.used <= 3


def test_state_slots():
    s = StateSlots(2)
    assert s.acquire("a") == 0 and s.acquire("b") == 1
    with pytest.raises(MemoryError):
        s.acquire("c")
    with pytest.raises(ValueError):
        s.acquire("a")
    s.release("a"); s.check()
    assert s.acquire("c") == 0
    s.check()


def test_state_is_zeroed_on_create_and_copied_on_fork():
    log = []
    m = CacheManager({0: KVNeed(1, 8)}, 4, 4, 3, state_needs={1: StateNeed((5,), "float32")},
                     allocate_state=lambda n, shape, dt: ("state", n, shape, dt),
                     zero_state=lambda t, s: log.append(("zero", s)), copy_state=lambda t, a, b: log.append(("copy", a, b)))
    assert m.state_storage[1] == ("state", 3, (5,), "float32")
    m.create("a"); m.fork("a", "b")
    assert log == [("zero", 0), ("copy", 0, 1)]
    (d,) = m.append_many([("b", 1)])
    assert d.state_slot == 1


@pytest.mark.parametrize("seed", range(6))
def test_random_orders_keep_every_page_accounted_for(seed):
    rng = random.Random(seed)
    m = manager(pages=12, page_size=4, sites=2, window=rng.choice([None, 3, 9]), max_requests=5)
    live, counter = {}, 0
    for _ in range(400):
        action = rng.random()
        if action < 0.25 and len(live) < 5:
            name = f"r{counter}"; counter += 1
            if live and rng.random() < 0.3:
                src = rng.choice(list(live))
                m.fork(src, name); live[name] = live[src]
            else:
                m.create(name); live[name] = 0
        elif action < 0.85 and live:
            picks = rng.sample(list(live), rng.randint(1, len(live)))
            items = [(r, rng.choice([1, 1, 1, 2, 5, 9])) for r in picks]
            snapshot = ({r: m.length(r) for r in live}, m.free_pages(),
                        [{r: list(t) for r, t in g.tables.items()} for g in m.groups])
            try:
                done = m.append_many(items)
            except OutOfPages:
                after = ({r: m.length(r) for r in live}, m.free_pages(),
                         [{r: list(t) for r, t in g.tables.items()} for g in m.groups])
                assert snapshot[0] == after[0], "a failed step changed a length"
                # a window may have given pages back (always valid); full groups are untouched
                for g, before_t, after_t in zip(m.groups, snapshot[2], after[2]):
                    if g.need.window is None:
                        assert before_t == after_t
                victim = rng.choice(list(live)); m.release(victim); del live[victim]
            else:
                for (r, n), d in zip(items, done):
                    assert d.start == live[r] and d.count == n
                    live[r] += n
                    for gid, g in enumerate(m.groups):
                        assert all(0 <= s < g.pool.n_pages * 4 for s in d.slots[gid])
                        assert len(set(d.slots[gid])) == n
                # no slot of this step is shared between two requests
                for gid in range(len(m.groups)):
                    flat = [s for d in done for s in d.slots[gid]]
                    assert len(flat) == len(set(flat))
        elif live:
            victim = rng.choice(list(live)); m.release(victim); del live[victim]
        m.check()
    for r in list(live):
        m.release(r)
    m.check()
    assert all(free == 12 for free in m.free_pages()) and len(m.slots.free) == 5


@pytest.mark.parametrize("seed", range(4))
def test_single_token_steps_take_the_same_pages_on_the_short_path(seed):
    """Steps of one token a request run a short path; it must hand out exactly the pages, slots, copies and
    errors of the general path, also after forks (shared last pages) and when the pool runs dry."""
    def run(fast):
        rng = random.Random(seed)
        copies = []
        m = CacheManager({0: KVNeed(2, 8, None), 1: KVNeed(2, 8, None), 2: KVNeed(1, 16, None)}, 10, 4, 6,
                         copy_pages=lambda group, pairs: copies.append(list(pairs)))
        m.fast_decode = fast
        live, counter, log = [], 0, []
        for _ in range(300):
            action = rng.random()
            if action < 0.2 and len(live) < 6:
                name = f"r{counter}"; counter += 1
                if live and rng.random() < 0.4:
                    m.fork(rng.choice(live), name)
                else:
                    m.create(name)
                    try:
                        m.append_many([(name, rng.choice([1, 3, 4, 6]))])     # a prompt portion: the general path
                    except OutOfPages:
                        pass
                live.append(name)
            elif action < 0.9 and live:
                picks = rng.sample(live, rng.randint(1, len(live)))
                try:
                    done = m.append_many([(r, 1) for r in picks])
                    log.append([(d.request, d.start, d.state_slot, dict(d.slots)) for d in done])
                except OutOfPages:
                    log.append("out of pages")
                    victim = rng.choice(live); m.release(victim); live.remove(victim)
            elif live:
                victim = rng.choice(live); m.release(victim); live.remove(victim)
            m.check()
        return log, copies, [dict(g.tables) for g in m.groups], [list(g.pool.free) for g in m.groups]

    assert run(True) == run(False)


def test_pages_that_fit_the_free_memory():
    from runtime.cache import KVNeed, pages_that_fit
    needs = {0: KVNeed(3, 64), 1: None, 2: KVNeed(3, 64), 3: KVNeed(2, 32, window=100)}
    per_page = 2 * 16 * 2 * (3 * 64 + 3 * 64 + 2 * 32)          # keys and values, 16 tokens, bf16
    assert pages_that_fit(needs, 16, 2, 10 * per_page, fraction=1.0) == 10
    assert pages_that_fit(needs, 16, 2, 10 * per_page) == 8                  # four fifths by default
    assert pages_that_fit(needs, 16, 4, 10 * per_page, fraction=1.0) == 5    # float32 pages are twice as large
    assert pages_that_fit(needs, 16, 2, 10 ** 12, most=777) == 777
    assert pages_that_fit({0: None}, 16, 2, 5) == 1                          # no site keeps keys: nothing to size
    with pytest.raises(MemoryError):
        pages_that_fit(needs, 16, 2, per_page - 1, fraction=1.0)


def test_fork_of_a_request_whose_window_has_passed_pages():
    """A fork copies the block tables as they are: the places of pages that a window has passed stay empty in the copy,
    the live pages are shared, the page being written is copied once by whoever writes first, and both requests go on
    giving pages back as their windows move."""
    window = KVNeed(1, 8, window=8)
    m = CacheManager({0: KVNeed(1, 8), 1: window}, {KVNeed(1, 8): 40, window: 12}, 4, 4)
    m.create("a")
    for n in (13, 1, 1, 9, 1):
        m.append_many([("a", n)])
        m.check()
    full, windowed = m.groups
    assert windowed.tables["a"][:4] == [-1] * 4 and all(p >= 0 for p in windowed.tables["a"][4:])
    m.fork("a", "b")
    m.check()
    assert windowed.tables["b"] == windowed.tables["a"] and full.tables["b"] == full.tables["a"]
    shared = [p for p in windowed.tables["a"] if p >= 0]
    assert all(windowed.pool.refs[p] == 2 for p in shared)
    for n in (1, 1, 6, 1):
        m.append_many([("a", n), ("b", n)])
        m.check()
    # position 25 was in a shared page of both groups: one of the two got a copy, the other kept the page
    assert full.tables["a"][6] != full.tables["b"][6] and full.tables["a"][:6] == full.tables["b"][:6]
    assert windowed.tables["a"].count(-1) == windowed.tables["b"].count(-1) == 6
    assert not set(p for p in windowed.tables["a"] if p >= 0) & set(p for p in windowed.tables["b"] if p >= 0)
    m.release("a"); m.check()
    m.release("b"); m.check()
    assert [g.pool.used for g in m.groups] == [0, 0]
