"""Cache manager: pages per group of layers, a block table per request and group,
and a slot per request for state of fixed size.

One *page group* per distinct need (all keys; a window of w keys).  Every layer of
a group shares the group's page ids and block tables; each group has its own
pool, so a windowed group never competes with an all-keys group for ids.  Rules
taken from the reference (inference_engine/block_manager.py:25-44,
inference_engine/scheduler.py:38-45,104-107): pages needed =
ceil((computed + n) / page) - len(table); reservation is all-or-nothing with an
optional watermark; everything a request holds goes back when it ends or is
preempted.  Beyond the reference: a windowed group also gives back pages that
lie wholly before the window once a step has passed them (their table entries
become 0, the scratch page), and every request holds a state slot.
"""
from __future__ import annotations

from dataclasses import dataclass, field

from .pages import CacheAccountingError, IdPool


@dataclass
class RequestCache:
    """What one live request holds."""
    request_id: object
    tables: list                     # per group: list of page ids, logical page -> physical (0 = released)
    first_live: list                 # per group: first logical page still held
    state_slot: int = 0
    closed: bool = False


@dataclass
class GroupSpec:
    window: int | None
    num_pages: int


class CacheManager:
    def __init__(self, page_size: int, groups: list[GroupSpec], num_state_slots: int):
        self.page_size = page_size
        self.groups = list(groups)
        self.pools = [IdPool(g.num_pages, 1, "page") for g in self.groups]
        self.slots = IdPool(num_state_slots, 1, "state slot")
        self.live: dict[object, RequestCache] = {}
        self.released_log: list = []     # (group, page) in release order, kept when keep_log is set
        self.keep_log = False
        self.on_release = None           # callable(group, pages), called as pages go back (debugging)
        self.on_open = None              # callable(slot), called as a state slot is handed to a request

    # ----------------------------------------------------------- lifecycle
    def can_open(self) -> bool:
        return self.slots.num_free > 0

    def open(self, request_id) -> RequestCache:
        if request_id in self.live:
            raise CacheAccountingError(f"request {request_id!r} is already open")
        slot = self.slots.take(1)
        if slot is None:
            raise CacheAccountingError("no state slot free")
        rc = RequestCache(request_id, [[] for _ in self.groups], [0 for _ in self.groups], slot[0])
        self.live[request_id] = rc
        if self.on_open is not None:
            self.on_open(slot[0])        # state of fixed size starts afresh with every request
        return rc

    def close(self, rc: RequestCache) -> None:
        if rc.closed:
            raise CacheAccountingError(f"request {rc.request_id!r} closed twice")
        for g, table in enumerate(rc.tables):
            self._release(g, [p for p in table if p != 0])
            rc.tables[g] = []
            rc.first_live[g] = 0
        self.slots.give_back([rc.state_slot])
        rc.state_slot = 0
        rc.closed = True
        del self.live[rc.request_id]

    def _release(self, g: int, pages: list[int]) -> None:
        self.pools[g].give_back(pages)
        if self.keep_log:
            self.released_log.extend((g, p) for p in pages)
        if self.on_release is not None and pages:
            self.on_release(g, pages)

    # ------------------------------------------------------------ reserving
    def pages_needed(self, rc: RequestCache, num_computed: int, n: int) -> list[int]:
        """Pages each group must add so that positions [num_computed, num_computed + n) have a slot."""
        total = -(-(num_computed + n) // self.page_size)
        return [max(0, total - len(t)) for t in rc.tables]

    def can_reserve(self, rc: RequestCache, num_computed: int, n: int, watermark: int = 0) -> bool:
        need = self.pages_needed(rc, num_computed, n)
        return all(k == 0 or pool.num_free - k >= watermark for pool, k in zip(self.pools, need))

    def reserve(self, rc: RequestCache, num_computed: int, n: int, watermark: int = 0) -> bool:
        """All groups or none (inference_engine/block_manager.py:32-40)."""
        if rc.closed:
            raise CacheAccountingError(f"request {rc.request_id!r} is closed")
        # most calls are a decoding request whose next token still fits its last page: nothing to do
        end = num_computed + n
        for t in rc.tables:
            if len(t) * self.page_size < end:
                break
        else:
            return True
        if not self.can_reserve(rc, num_computed, n, watermark):
            return False
        for g, k in enumerate(self.pages_needed(rc, num_computed, n)):
            if k:
                rc.tables[g].extend(self.pools[g].take(k))
        return True

    def advance(self, rc: RequestCache, num_computed: int) -> int:
        """After a step: ``num_computed`` tokens are in the cache.  Gives back the
        pages of windowed groups that no later query can see.  Returns how many."""
        freed = 0
        for g, spec in enumerate(self.groups):
            if spec.window is None:
                continue
            # the next query sits at position >= num_computed and sees keys >= num_computed - w + 1
            first = min(max(0, num_computed - spec.window + 1) // self.page_size, len(rc.tables[g]))
            gone = []
            for i in range(rc.first_live[g], first):
                if rc.tables[g][i] != 0:
                    gone.append(rc.tables[g][i])
                    rc.tables[g][i] = 0
            if first > rc.first_live[g]:
                rc.first_live[g] = first
            self._release(g, gone)
            freed += len(gone)
        return freed

    # ------------------------------------------------------------- queries
    def num_free(self, g: int = 0) -> int:
        return self.pools[g].num_free

    def usable_pages(self, g: int = 0) -> int:
        return self.pools[g].num_usable

    def max_tokens_one_request(self) -> int:
        """Longest request the all-keys groups can hold alone."""
        full = [p.num_usable for p, g in zip(self.pools, self.groups) if g.window is None]
        return min(full) * self.page_size if full else 1 << 62

    def check(self) -> None:
        """Invariants: every page is free, scratch, or in exactly one table."""
        for g, pool in enumerate(self.pools):
            seen = {}
            for rc in self.live.values():
                for p in rc.tables[g]:
                    if p == 0:
                        continue
                    if p in seen:
                        raise CacheAccountingError(f"group {g}: page {p} held by {seen[p]!r} and {rc.request_id!r}")
                    seen[p] = rc.request_id
            free = list(pool.free)
            if len(set(free)) != len(free):
                raise CacheAccountingError(f"group {g}: a page is on the free list twice")
            if set(free) & set(seen):
                raise CacheAccountingError(f"group {g}: pages both free and held: {sorted(set(free) & set(seen))}")
            if len(free) + len(seen) + pool.reserved != pool.count:
                raise CacheAccountingError(
                    f"group {g}: {len(free)} free + {len(seen)} held + {pool.reserved} scratch != {pool.count}")
            if pool.held() != set(seen):
                raise CacheAccountingError(f"group {g}: pool and tables disagree on what is held")
        slots = [rc.state_slot for rc in self.live.values()]
        if len(set(slots)) != len(slots) or 0 in slots:
            raise CacheAccountingError("state slots: held twice or scratch handed out")
        if len(slots) + self.slots.num_free + 1 != self.slots.count:
            raise CacheAccountingError("state slots lost")
