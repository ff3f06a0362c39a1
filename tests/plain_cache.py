"""A plain cache manager in Python, for the tests: the same rules as the engine's (C++) one,
written down separately, so that the two can be run side by side on random orders of requests.

The cache manager: pages, block tables and state slots, kept on the host.

Reference: `BlockManager` hands out block ids from a FIFO free list and a
`PagedKVCache` grows a per-sequence block table as positions cross block
boundaries, giving everything back at `release_all` (src/paged_kv.cpp:8-47,
88-101,135-139). Here the same bookkeeping is done before a step instead of
inside the forward pass: pages for all tokens of a step are reserved first, so a
step never fails for capacity half-way.

Layers with the same needs form a group with a page pool and block tables of its
own: a "full" group keeps every token of a request; a "window" group gives pages
back once every position in them lies behind the window of the next token. Beside
the pages, every live request holds a slot: a row in each fixed-size state tensor.
"""
from __future__ import annotations

from collections import deque
from dataclasses import dataclass, field


class CacheError(RuntimeError):
    pass


class PagePool:
    """A fixed set of page ids; FIFO reuse like the reference's free list
    (src/paged_kv.cpp:30-42). Freeing a page that is not held raises."""

    def __init__(self, num_pages: int):
        if num_pages <= 0:
            raise ValueError("a page pool needs at least one page")
        self.num_pages = int(num_pages)
        self._free: deque[int] = deque(range(self.num_pages))
        self._held: set[int] = set()

    @property
    def free_pages(self) -> int:
        return len(self._free)

    def allocate(self) -> int | None:
        if not self._free:
            return None
        page = self._free.popleft()
        self._held.add(page)
        return page

    def free(self, page: int) -> None:
        if page not in self._held:
            raise CacheError(f"page {page} is freed but not held")
        self._held.remove(page)
        self._free.append(page)

    def held(self) -> set[int]:
        return set(self._held)


@dataclass(frozen=True)
class GroupSpec:
    name: str
    kind: str = "full"          # "full" | "window"
    window: int = 0
    num_pages: int = 0


@dataclass
class _Request:
    slot: int
    length: int = 0                                             # tokens committed
    reserved: int = 0                                           # tokens with pages reserved (>= length)
    tables: dict[str, list[int]] = field(default_factory=dict)  # group -> page per logical block, -1 = given back


class CacheManager:
    def __init__(self, groups: list[GroupSpec], page_size: int, max_requests: int):
        if page_size <= 0:
            raise ValueError("page_size must be >= 1")
        if max_requests <= 0:
            raise ValueError("max_requests must be >= 1")
        names = [g.name for g in groups]
        if len(set(names)) != len(names):
            raise ValueError(f"cache groups must have distinct names, got {names}")
        for g in groups:
            if g.kind not in ("full", "window"):
                raise ValueError(f"group {g.name}: kind {g.kind!r} is not 'full' or 'window'")
            if g.kind == "window" and g.window <= 0:
                raise ValueError(f"group {g.name}: a window group needs window > 0")
        self.page_size = int(page_size)
        self.max_requests = int(max_requests)
        self.groups = {g.name: g for g in groups}
        self.pools = {g.name: PagePool(g.num_pages) for g in groups}
        self._free_slots: list[int] = list(range(self.max_requests - 1, -1, -1))
        self._requests: dict[object, _Request] = {}

    # ---- requests and slots ----
    def admit(self, request_id) -> int:
        if request_id in self._requests:
            raise CacheError(f"request {request_id!r} is already live")
        if not self._free_slots:
            raise CacheError(f"no free slot: {self.max_requests} requests are live")
        slot = self._free_slots.pop()
        self._requests[request_id] = _Request(slot=slot, tables={g: [] for g in self.groups})
        return slot

    def is_live(self, request_id) -> bool:
        return request_id in self._requests

    def live_requests(self) -> list:
        return list(self._requests)

    def slot(self, request_id) -> int:
        return self._req(request_id).slot

    def length(self, request_id) -> int:
        return self._req(request_id).length

    def free_slots(self) -> int:
        return len(self._free_slots)

    def _req(self, request_id) -> _Request:
        try:
            return self._requests[request_id]
        except KeyError:
            raise CacheError(f"request {request_id!r} is not live") from None

    # ---- pages ----
    def _first_needed_block(self, group: GroupSpec, position: int) -> int:
        """First logical block that a token at `position` reads in this group."""
        if group.kind == "window":
            return max(0, position - group.window + 1) // self.page_size
        return 0

    def _missing(self, req: _Request, group: GroupSpec, n_new: int) -> list[int]:
        """Logical blocks that must get a page before n_new tokens are appended."""
        table = req.tables[group.name]
        start, end = req.length, req.length + n_new
        first = self._first_needed_block(group, start)
        last = (end - 1) // self.page_size
        return [b for b in range(first, last + 1) if b >= len(table) or table[b] < 0]

    def pages_needed(self, request_id, n_new: int) -> dict[str, int]:
        req = self._req(request_id)
        return {g.name: len(self._missing(req, g, n_new)) for g in self.groups.values()}

    def can_reserve(self, request_id, n_new: int, pending: dict[str, int] | None = None) -> bool:
        """True if pages for n_new more tokens are free; `pending` counts pages that
        other reservations of the same step will take first."""
        for name, need in self.pages_needed(request_id, n_new).items():
            if need + (pending or {}).get(name, 0) > self.pools[name].free_pages:
                return False
        return True

    def reserve(self, request_id, n_new: int) -> bool:
        """Gives the request pages for positions [length, length + n_new) in every
        group, or changes nothing and returns False if any pool is short."""
        if n_new <= 0:
            raise ValueError("reserve needs n_new >= 1")
        req = self._req(request_id)
        missing = {g.name: self._missing(req, g, n_new) for g in self.groups.values()}
        for name, blocks in missing.items():
            if len(blocks) > self.pools[name].free_pages:
                return False
        for name, blocks in missing.items():
            table = req.tables[name]
            for b in blocks:
                while len(table) <= b:
                    table.append(-1)
                page = self.pools[name].allocate()
                assert page is not None
                table[b] = page
        req.reserved = max(req.reserved, req.length + n_new)
        return True

    def reserve_batch(self, items: list[tuple[object, int]]) -> bool:
        """`reserve` for several requests at once: all of them get their pages, or nothing changes."""
        plans = []
        need = {name: 0 for name in self.groups}
        for request_id, n_new in items:
            if n_new <= 0:
                raise ValueError("reserve needs n_new >= 1")
            req = self._req(request_id)
            last = (req.length + n_new - 1) // self.page_size
            for g in self.groups.values():
                table = req.tables[g.name]
                if g.kind == "full":
                    if last < len(table):
                        continue                    # the common case of decoding: the page is there
                    blocks = list(range(len(table), last + 1))
                else:
                    blocks = self._missing(req, g, n_new)
                    if not blocks:
                        continue
                need[g.name] += len(blocks)
                plans.append((req, g.name, blocks))
        for name, n in need.items():
            if n > self.pools[name].free_pages:
                return False
        for req, name, blocks in plans:
            table = req.tables[name]
            pool = self.pools[name]
            for b in blocks:
                while len(table) <= b:
                    table.append(-1)
                table[b] = pool.allocate()
        for request_id, n_new in items:
            req = self._requests[request_id]
            req.reserved = max(req.reserved, req.length + n_new)
        return True

    def commit(self, request_id, n_new: int) -> None:
        """The step wrote n_new tokens: the request is that much longer, and window
        groups give back the pages no later token will read."""
        req = self._req(request_id)
        if req.length + n_new > req.reserved:
            raise CacheError(f"request {request_id!r}: commit of {n_new} tokens beyond the reserved pages")
        req.length += n_new
        for g in self.groups.values():
            if g.kind != "window":
                continue
            table = req.tables[g.name]
            keep_from = self._first_needed_block(g, req.length)     # next token's first block
            for b in range(min(keep_from, len(table))):
                if table[b] >= 0:
                    self.pools[g.name].free(table[b])
                    table[b] = -1

    def release(self, request_id) -> None:
        """The request is over: all its pages and its slot are given back."""
        req = self._req(request_id)
        for name, table in req.tables.items():
            for page in table:
                if page >= 0:
                    self.pools[name].free(page)
        self._free_slots.append(req.slot)
        del self._requests[request_id]

    def block_table(self, request_id, group: str) -> list[int]:
        return self._req(request_id).tables[group]

    def free_pages(self, group: str | None = None) -> int:
        if group is None:
            if len(self.pools) != 1:
                raise ValueError("name the group: there are several")
            group = next(iter(self.pools))
        return self.pools[group].free_pages

    def num_pages(self, group: str | None = None) -> int:
        if group is None:
            if len(self.pools) != 1:
                raise ValueError("name the group: there are several")
            group = next(iter(self.pools))
        return self.pools[group].num_pages

    # ---- invariants, for tests and debugging ----
    def check(self) -> None:
        """No page is lost or held twice, no slot is held twice."""
        for name, pool in self.pools.items():
            owned: list[int] = []
            for req in self._requests.values():
                owned += [p for p in req.tables[name] if p >= 0]
            if len(owned) != len(set(owned)):
                raise CacheError(f"group {name}: a page is in two block tables")
            if set(owned) != pool.held():
                raise CacheError(f"group {name}: pages held {sorted(pool.held())} != pages in tables {sorted(owned)}")
            if len(owned) + pool.free_pages != pool.num_pages:
                raise CacheError(f"group {name}: {pool.num_pages - len(owned) - pool.free_pages} pages lost")
        slots = [r.slot for r in self._requests.values()]
        if len(slots) != len(set(slots)) or set(slots) & set(self._free_slots):
            raise CacheError("a slot is held twice")
        if len(slots) + len(self._free_slots) != self.max_requests:
            raise CacheError("a slot is lost")
