"""The cache manager's bookkeeping (no GPU): pages are never lost, held twice or freed
twice, under random orders of requests; window groups give pages back as the window passes;
slots are unique; reservation is all-or-nothing."""
import random

import pytest

from llmengine.cache import CacheError, CacheManager, GroupSpec, PagePool


def test_pool_fifo_and_double_free():
    pool = PagePool(3)
    a, b, c = pool.allocate(), pool.allocate(), pool.allocate()
    assert (a, b, c) == (0, 1, 2) and pool.allocate() is None and pool.free_pages == 0
    pool.free(b)
    pool.free(a)
    assert pool.allocate() == b and pool.allocate() == a          # first freed, first reused
    with pytest.raises(CacheError):
        pool.free(7)
    pool.free(c)
    with pytest.raises(CacheError):
        pool.free(c)                                               # freed twice


def test_pages_follow_token_counts():
    m = CacheManager([GroupSpec("full", "full", 0, 8)], page_size=4, max_requests=2)
    m.admit("a")
    assert m.pages_needed("a", 9) == {"full": 3}                   # 9 tokens at 4 a page: 3 pages
    assert m.reserve("a", 9)
    m.commit("a", 9)
    assert m.free_pages() == 5 and len(m.block_table("a", "full")) == 3
    assert m.pages_needed("a", 3) == {"full": 0}                   # tokens 9..11 fit the third page
    assert m.pages_needed("a", 4) == {"full": 1}
    m.release("a")
    assert m.free_pages() == 8
    m.check()


def test_reservation_is_all_or_nothing():
    m = CacheManager([GroupSpec("full", "full", 0, 1)], page_size=4, max_requests=2)
    m.admit("a")
    assert not m.reserve("a", 6)                                   # needs 2 pages, 1 is there
    assert m.free_pages() == 1 and m.block_table("a", "full") == []
    assert m.reserve("a", 4)
    m.commit("a", 4)
    assert not m.can_reserve("a", 1)                               # position 4 needs a second page
    with pytest.raises(CacheError):
        m.commit("a", 1)                                           # nothing was reserved for it
    m.release("a")
    assert m.free_pages() == 1


def test_pending_counts_against_free_pages():
    m = CacheManager([GroupSpec("full", "full", 0, 3)], page_size=4, max_requests=4)
    m.admit("a")
    m.admit("b")
    assert m.can_reserve("a", 8) and m.can_reserve("b", 8)
    assert not m.can_reserve("b", 8, pending={"full": 2})


def test_window_group_gives_pages_back():
    m = CacheManager([GroupSpec("full", "full", 0, 64), GroupSpec("win", "window", 6, 64)],
                     page_size=4, max_requests=1)
    m.admit("r")
    assert m.reserve("r", 10)
    m.commit("r", 10)                      # next token at 10 reads keys 5..10: block 0 (keys 0..3) is behind
    assert m.block_table("r", "win")[0] == -1 and m.block_table("r", "win")[1] >= 0
    assert m.block_table("r", "full")[0] >= 0
    for _ in range(30):
        assert m.reserve("r", 1)
        m.commit("r", 1)
        m.check()
    live = [p for p in m.block_table("r", "win") if p >= 0]
    assert len(live) <= 3                                          # a 6-token window spans at most 3 pages of 4
    assert len([p for p in m.block_table("r", "full") if p >= 0]) == 10
    # a long portion needs pages for all its own tokens, but none behind the window of its first
    assert m.pages_needed("r", 9)["win"] == len(range(40 // 4, (40 + 9 - 1) // 4 + 1)) - 0
    m.release("r")
    assert m.free_pages("win") == 64 and m.free_pages("full") == 64


def test_slots():
    m = CacheManager([GroupSpec("full", "full", 0, 4)], page_size=4, max_requests=2)
    s0, s1 = m.admit("a"), m.admit("b")
    assert {s0, s1} == {0, 1}
    with pytest.raises(CacheError):
        m.admit("c")
    with pytest.raises(CacheError):
        m.admit("a")
    m.release("a")
    assert m.admit("c") == s0
    with pytest.raises(CacheError):
        m.release("a")
    with pytest.raises(CacheError):
        m.length("zzz")


@pytest.mark.parametrize("seed", range(8))
def test_random_orders_keep_the_invariants(seed):
    rng = random.Random(seed)
    groups = [GroupSpec("full", "full", 0, 40)]
    if seed % 2:
        groups.append(GroupSpec("win", "window", rng.choice([3, 8, 17]), 25))
    m = CacheManager(groups, page_size=rng.choice([1, 4, 16]), max_requests=5)
    live: dict[int, int] = {}
    next_id = 0
    for _ in range(600):
        op = rng.random()
        if op < 0.25 and m.free_slots():
            m.admit(next_id)
            live[next_id] = 0
            next_id += 1
        elif op < 0.85 and live:
            rid = rng.choice(list(live))
            n = rng.choice([1, 1, 1, 2, 5, 9, 33])
            before = {g: m.free_pages(g) for g in m.groups}
            tables = {g: list(m.block_table(rid, g)) for g in m.groups}
            if m.reserve(rid, n):
                assert m.can_reserve(rid, n)                      # now nothing more is needed
                m.commit(rid, n)
                live[rid] += n
                assert m.length(rid) == live[rid]
            else:
                assert before == {g: m.free_pages(g) for g in m.groups}     # a refusal changes nothing
                assert tables == {g: list(m.block_table(rid, g)) for g in m.groups}
        elif live:
            rid = rng.choice(list(live))
            m.release(rid)
            del live[rid]
        m.check()
        for rid, n in live.items():                               # every readable key has a page
            for g in m.groups.values():
                table = m.block_table(rid, g.name)
                lo = max(0, n - g.window + 1) if g.kind == "window" else 0   # the next token at n reads keys > n - window
                for pos in range(lo, n):
                    assert table[pos // m.page_size] >= 0
    for rid in list(live):
        m.release(rid)
    m.check()
    assert all(m.free_pages(g) == m.num_pages(g) for g in m.groups)


def test_bad_arguments():
    with pytest.raises(ValueError):
        CacheManager([GroupSpec("g", "full", 0, 4)], page_size=0, max_requests=1)
    with pytest.raises(ValueError):
        CacheManager([GroupSpec("g", "window", 0, 4)], page_size=4, max_requests=1)
    with pytest.raises(ValueError):
        CacheManager([GroupSpec("g", "full", 0, 4), GroupSpec("g", "full", 0, 4)], page_size=4, max_requests=1)
    with pytest.raises(ValueError):
        PagePool(0)


def test_reserve_batch_is_all_or_nothing():
    m = CacheManager([GroupSpec("full", "full", 0, 6), GroupSpec("win", "window", 6, 6)], page_size=4, max_requests=3)
    for r in "abc":
        m.admit(r)
    assert m.reserve_batch([("a", 8), ("b", 4)])                       # 2 + 1 pages in each group
    m.commit("a", 8)
    m.commit("b", 4)
    m.check()
    before = {g: m.free_pages(g) for g in m.groups}
    tables = {r: list(m.block_table(r, "full")) for r in "abc"}
    assert not m.reserve_batch([("a", 1), ("c", 12)])                  # a needs 1, c needs 3: 4 > 3 free
    assert before == {g: m.free_pages(g) for g in m.groups}
    assert tables == {r: list(m.block_table(r, "full")) for r in "abc"}
    assert m.reserve_batch([("a", 1), ("b", 1), ("c", 4)])             # a and b: a new page each; c: one
    for r, n in (("a", 1), ("b", 1), ("c", 4)):
        m.commit(r, n)
    m.check()
    assert m.reserve_batch([("a", 3)])                                  # tokens 9..11 fit a's third page
    assert m.free_pages("full") == 6 - 3 - 2 - 1                        # a 3 pages, b 2, c 1
    with pytest.raises(ValueError):
        m.reserve_batch([("a", 0)])


@pytest.mark.parametrize("seed", range(6))
def test_native_manager_agrees_with_the_plain_one(seed):
    """The C++ manager and the plain Python one, fed the same random requests, give the same
    answers at every turn: slots, lengths, pages needed, refusals, block tables, free pages."""
    import plain_cache
    rng = random.Random(100 + seed)
    specs = [("full", "full", 0, rng.choice([9, 30])), ("win", "window", rng.choice([2, 7, 20]), rng.choice([6, 18]))]
    if seed % 3 == 0:
        specs = specs[:1]
    page = rng.choice([1, 4, 16])
    a = CacheManager([GroupSpec(*s) for s in specs], page, 4)
    b = plain_cache.CacheManager([plain_cache.GroupSpec(*s) for s in specs], page, 4)
    live, next_id = [], 0
    for _ in range(500):
        op = rng.random()
        if op < 0.2 and a.free_slots():
            rid = next_id if next_id % 2 else f"r{next_id}"         # integer and other names
            next_id += 1
            assert a.admit(rid) == b.admit(rid)
            live.append(rid)
        elif op < 0.8 and live:
            items = [(rid, rng.choice([1, 1, 2, 6, 19])) for rid in rng.sample(live, rng.randint(1, len(live)))]
            for rid, n in items:
                assert a.pages_needed(rid, n) == b.pages_needed(rid, n)
                pending = {g: rng.randint(0, 3) for g in a.groups}
                assert a.can_reserve(rid, n, pending) == b.can_reserve(rid, n, pending)
            ok = a.reserve_batch(items)
            assert ok == b.reserve_batch(items)
            if ok:
                for rid, n in items:
                    a.commit(rid, n)
                    b.commit(rid, n)
        elif live:
            rid = live.pop(rng.randrange(len(live)))
            a.release(rid)
            b.release(rid)
        a.check()
        assert a.free_slots() == b.free_slots() and a.live_requests() == b.live_requests()
        for g in a.groups:
            assert a.free_pages(g) == b.free_pages(g)
        for rid in live:
            assert (a.slot(rid), a.length(rid)) == (b.slot(rid), b.length(rid))
            for g in a.groups:
                assert a.block_table(rid, g) == b.block_table(rid, g)


def test_decode_begin_checks_the_position_limit_before_it_reserves():
    """The decode step's one call for lengths, limit and pages: a request that would pass the
    position limit stops the call before any page is reserved for any request of the batch."""
    import ctypes
    m = CacheManager([GroupSpec("full", "full", 0, 8)], 4, 3)
    for rid, n in ((0, 4), (1, 8), (2, 3)):             # requests 0 and 1 need a new page for their next token
        m.admit(rid)
        assert m.reserve(rid, n)
        m.commit(rid, n)
    free = m.free_pages()
    keys = (ctypes.c_int64 * 3)(*[m.key_of(r) for r in (0, 1, 2)])
    lengths = (ctypes.c_int * 3)()
    assert m._lib.llme_cm_decode_begin(m.handle, 3, keys, lengths, 8) == 2       # request 1 would be 9 long
    assert list(lengths) == [4, 8, 3] and m.free_pages() == free
    m.check()
    assert m._lib.llme_cm_decode_begin(m.handle, 3, keys, lengths, 9) == 1
    assert m.free_pages() == free - 2
    assert m._lib.llme_cm_commit_batch(m.handle, 3, keys, 1) == 0
    m.check()
    assert m._lib.llme_cm_decode_begin(m.handle, 3, keys, lengths, 0) == 1       # 0: no limit


def test_a_steps_integer_arrays_are_what_the_manager_knows():
    """The arrays a step hands to the kernels (positions, request index per token, first rows,
    lengths, slots, block tables by group, wanted rows) as the C++ manager writes them in one call,
    against the same arrays put together here from the manager's single answers, for random
    batches over a full and a window group, with pages given back and used again."""
    import random
    import numpy as np
    from llmengine.engine.step import StepEntry, fill_step_arrays, step_layout
    rng = random.Random(5)
    page = 4
    mgr = CacheManager([GroupSpec("full", "full", 0, 1200), GroupSpec("window8", "window", 8, 200)], page, 12)
    live = {}
    for step_no in range(200):
        for rid in [r for r, n in live.items() if n > 250 or rng.random() < 0.05]:
            mgr.release(rid)
            del live[rid]
        while len(live) < 2 or (len(live) < 12 and rng.random() < 0.3):
            rid = rng.choice([f"r{step_no}_{len(live)}", 1000 * step_no + len(live)])      # text and integer ids
            mgr.admit(rid)
            live[rid] = 0
        chosen = rng.sample(sorted(live, key=str), rng.randint(1, len(live)))
        entries = []
        for rid in chosen:
            n = rng.choice([1, 1, 1, 2, 5, 9, 23])
            toks = [rng.randrange(50) for _ in range(n)]
            entries.append(StepEntry(rid, toks, sorted(rng.sample(range(n), rng.randint(0, min(n, 3))))))
        assert mgr.reserve_batch([(e.request_id, len(e.tokens)) for e in entries])
        for width in (None, 40):
            layout = step_layout(mgr, entries, page, width)
            new_lens, ctx_lens, max_blocks, offsets, sizes, total, T, R = layout[:8]
            h = np.full(total + 5, -9, dtype=np.int32)
            slots, top = fill_step_arrays(mgr, entries, layout, h)
            assert (h[total:] == -9).all()
            # the same from single answers
            want = np.zeros(total, dtype=np.int32)
            pos, r0 = 0, 0
            for i, e in enumerate(entries):
                n, c = len(e.tokens), mgr.length(e.request_id)
                want[offsets[0] + pos:offsets[0] + pos + n] = e.tokens
                want[offsets[1] + pos:offsets[1] + pos + n] = range(c, c + n)
                want[offsets[2] + pos:offsets[2] + pos + n] = i
                want[offsets[3] + i] = pos
                want[offsets[4] + i] = c
                want[offsets[5] + i] = mgr.slot(e.request_id)
                for gi, g in enumerate(mgr.groups):
                    table = mgr.block_table(e.request_id, g)[:max_blocks]
                    at = offsets[6 + gi] + i * max_blocks
                    want[at:at + len(table)] = table
                want[offsets[-2] + r0:offsets[-2] + r0 + len(e.want)] = [pos + w for w in e.want]
                r0 += len(e.want)
                pos += n
            want[offsets[3] + len(entries)] = pos
            assert np.array_equal(h[:total], want), (step_no, width)
            assert ctx_lens == [mgr.length(e.request_id) for e in entries]
            assert slots == [mgr.slot(e.request_id) for e in entries]
            assert top == max(c + n for c, n in zip(ctx_lens, new_lens)) - 1 and T == pos and R == r0
        for e in entries:
            mgr.commit(e.request_id, len(e.tokens))
            live[e.request_id] += len(e.tokens)
        mgr.check()
