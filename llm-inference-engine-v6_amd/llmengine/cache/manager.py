"""The cache manager: pages, block tables and state slots, kept on the host.

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

The bookkeeping itself is C++ (csrc/host/cache_manager.cpp); the classes here name
groups and requests (any hashable; the C++ side knows them by 64-bit keys) and turn
its codes into exceptions.
"""
from __future__ import annotations

import ctypes
from dataclasses import dataclass

from ..runtime import native


class CacheError(RuntimeError):
    pass


class PagePool:
    """A fixed set of page ids; FIFO reuse like the reference's free list
    (src/paged_kv.cpp:30-42). Freeing a page that is not held raises."""

    def __init__(self, num_pages: int):
        if num_pages <= 0:
            raise ValueError("a page pool needs at least one page")
        self.num_pages = int(num_pages)
        self._lib = native.library()
        self._h = self._lib.llme_pool_create(self.num_pages)

    def __del__(self):
        if getattr(self, "_h", None):
            self._lib.llme_pool_destroy(self._h)
            self._h = None

    @property
    def free_pages(self) -> int:
        return self._lib.llme_pool_free_pages(self._h)

    def allocate(self) -> int | None:
        page = self._lib.llme_pool_allocate(self._h)
        return None if page < 0 else page

    def free(self, page: int) -> None:
        if self._lib.llme_pool_free(self._h, int(page)) != 0:
            raise CacheError(f"page {page} is freed but not held")

    def held(self) -> set[int]:
        return {p for p in range(self.num_pages) if self._lib.llme_pool_is_held(self._h, p)}


@dataclass(frozen=True)
class GroupSpec:
    name: str
    kind: str = "full"          # "full" | "window"
    window: int = 0
    num_pages: int = 0


_TEXT_KEYS = 1 << 62            # keys of requests that are not named by a small integer


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
            if g.num_pages <= 0:
                raise ValueError("a page pool needs at least one page")
        self.page_size = int(page_size)
        self.max_requests = int(max_requests)
        self.groups = {g.name: g for g in groups}
        self._index = {g.name: i for i, g in enumerate(groups)}
        self._lib = native.library()
        n = len(groups)
        arr = ctypes.c_int * max(n, 1)
        self._h = self._lib.llme_cm_create(n, arr(*[int(g.kind == "window") for g in groups]),
                                           arr(*[int(g.window) for g in groups]),
                                           arr(*[int(g.num_pages) for g in groups]), self.page_size, self.max_requests)
        if not self._h:
            raise ValueError("the cache manager refused its sizes")
        self._keys: dict[object, int] = {}          # request id -> key on the C++ side
        self._ids: dict[int, object] = {}
        self._next_key = _TEXT_KEYS
        self._counts = arr()

    def __del__(self):
        if getattr(self, "_h", None):
            self._lib.llme_cm_destroy(self._h)
            self._h = None

    @property
    def handle(self) -> int:
        """The C++ object, for the other parts of the host runtime (the scheduler)."""
        return self._h

    # ---- names ----
    def key_of(self, request_id, create: bool = False) -> int:
        """The 64-bit key of a request: a non-negative integer below 2^62 is its own key (so a
        request that the C++ scheduler admitted under its sequence id is found by that id),
        anything else gets a key of its own while it is live."""
        if isinstance(request_id, int) and not isinstance(request_id, bool) and 0 <= request_id < _TEXT_KEYS:
            return request_id
        key = self._keys.get(request_id)
        if key is None and create:
            key = self._next_key
            self._next_key += 1
        return -1 if key is None else key

    def _key(self, request_id) -> int:
        key = self.key_of(request_id)
        if key < 0 or not self._lib.llme_cm_is_live(self._h, key):
            raise CacheError(f"request {request_id!r} is not live")
        return key

    def _group(self, group: str | None) -> int:
        if group is None:
            if len(self.groups) != 1:
                raise ValueError("name the group: there are several")
            return 0
        return self._index[group]

    # ---- requests and slots ----
    def admit(self, request_id) -> int:
        key = self.key_of(request_id, create=True)
        slot = self._lib.llme_cm_admit(self._h, key)
        if slot == native.ALREADY_LIVE:
            raise CacheError(f"request {request_id!r} is already live")
        if slot == native.NO_SLOT:
            raise CacheError(f"no free slot: {self.max_requests} requests are live")
        if key >= _TEXT_KEYS:
            self._keys[request_id] = key
            self._ids[key] = request_id
        return slot

    def is_live(self, request_id) -> bool:
        key = self.key_of(request_id)
        return key >= 0 and bool(self._lib.llme_cm_is_live(self._h, key))

    def live_requests(self) -> list:
        buf = (ctypes.c_int64 * self.max_requests)()
        n = self._lib.llme_cm_live(self._h, buf, self.max_requests)
        return [self._ids.get(buf[i], buf[i]) for i in range(n)]

    def slot(self, request_id) -> int:
        return self._lib.llme_cm_slot(self._h, self._key(request_id))

    def length(self, request_id) -> int:
        return self._lib.llme_cm_length(self._h, self._key(request_id))

    def free_slots(self) -> int:
        return self._lib.llme_cm_free_slots(self._h)

    # ---- pages ----
    def pages_needed(self, request_id, n_new: int) -> dict[str, int]:
        self._lib.llme_cm_pages_needed(self._h, self._key(request_id), int(n_new), self._counts)
        return {name: self._counts[i] for name, i in self._index.items()}

    def can_reserve(self, request_id, n_new: int, pending: dict[str, int] | None = None) -> bool:
        """True if pages for n_new more tokens are free; `pending` counts pages that
        other reservations of the same step will take first."""
        arr = None
        if pending:
            arr = (ctypes.c_int * max(len(self.groups), 1))(*[int(pending.get(name, 0)) for name in self.groups])
        return self._lib.llme_cm_can_reserve(self._h, self._key(request_id), int(n_new), arr) == 1

    def reserve(self, request_id, n_new: int) -> bool:
        """Gives the request pages for positions [length, length + n_new) in every
        group, or changes nothing and returns False if any pool is short."""
        return self.reserve_batch([(request_id, n_new)])

    def reserve_batch(self, items: list[tuple[object, int]]) -> bool:
        """`reserve` for several requests at once: all of them get their pages, or nothing changes."""
        n = len(items)
        for _, n_new in items:
            if n_new <= 0:
                raise ValueError("reserve needs n_new >= 1")
        keys = (ctypes.c_int64 * max(n, 1))(*[self._key(r) for r, _ in items])
        counts = (ctypes.c_long * max(n, 1))(*[int(k) for _, k in items])
        rc = self._lib.llme_cm_reserve_batch(self._h, n, keys, counts)
        if rc < 0:
            raise ValueError("reserve_batch: a request appears twice")
        return rc == 1

    def commit(self, request_id, n_new: int) -> None:
        """The step wrote n_new tokens: the request is that much longer, and window
        groups give back the pages no later token will read."""
        rc = self._lib.llme_cm_commit(self._h, self._key(request_id), int(n_new))
        if rc == native.NOT_RESERVED:
            raise CacheError(f"request {request_id!r}: commit of {n_new} tokens beyond the reserved pages")

    def release(self, request_id) -> None:
        """The request is over: all its pages and its slot are given back."""
        key = self._key(request_id)
        self._lib.llme_cm_release(self._h, key)
        if key >= _TEXT_KEYS:
            self._keys.pop(self._ids.pop(key), None)

    def forget(self, request_id) -> None:
        """Drops the name of a request that the C++ side has released on its own."""
        key = self._keys.pop(request_id, None)
        if key is not None:
            self._ids.pop(key, None)

    def block_table(self, request_id, group: str) -> list[int]:
        key, g = self._key(request_id), self._index[group]
        n = self._lib.llme_cm_table_len(self._h, key, g)
        buf = (ctypes.c_int * max(n, 1))()
        self._lib.llme_cm_table_copy(self._h, key, g, 0, n, buf)
        return list(buf[:n])

    def free_pages(self, group: str | None = None) -> int:
        return self._lib.llme_cm_free_pages(self._h, self._group(group))

    def num_pages(self, group: str | None = None) -> int:
        return self._lib.llme_cm_num_pages(self._h, self._group(group))

    # ---- invariants, for tests and debugging ----
    def check(self) -> None:
        """No page is lost or held twice, no slot is held twice."""
        rc = self._lib.llme_cm_check(self._h)
        if rc != 0:
            raise CacheError(native.CHECK_MESSAGES.get(rc, f"inconsistent (code {rc})"))
