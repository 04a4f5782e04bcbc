"""The cache manager: paged keys and values with a block table per request,
one pool per group of runs with the same needs, and slots of fixed size for
per-request state.

What a run (an entry of the model's execution order) needs is said by its
mixer as a cache spec (``cache/specs.py``): something for every token, in pages
(with a window, pages wholly below it are given back while the request still
runs), or one array of fixed shape per request, or ``None`` (nothing, or the
run reads another run's cache).  The manager asks a spec what it stores, how
much, and what view a run gets; it holds no knowledge of keys and values.

Runs with equal per-token specs form a group: one page pool and one block
table per request serve all of them, and page ``p`` means slice ``p`` of every
run of the group (reference: src/runtime/kv_cache_manager.cpp:56-76, one group
of all layers; growth and release there: :83-173, :175-204).  Groups with
different needs have pools, page ids and storage of their own.

All bookkeeping is host code and is exact: a page is handed out once, returned
once.  Pages for a step are reserved before the step runs; the step itself
never allocates.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Dict, Hashable, List, Optional, Sequence, Tuple

from .page_pool import OutOfPages, PageError, PagePool
from .specs import PagedKVSpec, StateSpec, check_spec  # noqa: F401  (the two specs are part of this module's names)


class CacheError(RuntimeError):
    pass


class StateSlots:
    """Slot numbers for live requests; slot ``s`` addresses row ``s`` of every per-request array."""

    def __init__(self, num_slots: int):
        if num_slots <= 0:
            raise ValueError("at least one state slot is needed")
        self.num_slots = int(num_slots)
        self._free = list(range(self.num_slots - 1, -1, -1))
        self._owner: Dict[int, Hashable] = {}

    @property
    def num_free(self) -> int:
        return len(self._free)

    def take(self, owner: Hashable) -> int:
        if not self._free:
            raise CacheError(f"all {self.num_slots} request slots are in use")
        slot = self._free.pop()
        self._owner[slot] = owner
        return slot

    def give_back(self, slot: int) -> None:
        if slot not in self._owner:
            raise CacheError(f"slot {slot} is not in use")
        del self._owner[slot]
        self._free.append(slot)


@dataclass
class CacheGroup:
    """Runs that share a page pool and block tables."""

    index: int
    spec: Any              # the per-token cache spec that all its runs share
    page_size: int
    runs: List[int]
    pool: PagePool
    tables: Dict[Hashable, List[int]] = field(default_factory=dict)  # -1: page given back (below the window)
    storage: Any = None    # what the spec allocated for all runs of the group

    @property
    def window(self) -> Optional[int]:
        return getattr(self.spec, "window", None)

    def pages_for(self, length: int) -> int:
        return (length + self.page_size - 1) // self.page_size

    def first_needed_token(self, computed: int) -> int:
        """The lowest key position that a token at position >= computed can still read."""
        if self.window is None:
            return 0
        return max(0, computed - self.window + 1)


@dataclass
class _Request:
    slot: int
    computed: int = 0   # tokens whose keys are in the cache
    reserved: int = 0   # tokens that pages are reserved for
    capacity: int = 0   # tokens that the pages it has can hold (the fewest over the groups)
    stamp: int = 0      # changes whenever one of its block tables does (never the same for two requests)


class CacheManager:
    def __init__(self, run_specs: Sequence[object], page_size: int, num_pages: int, max_requests: int,
                 group_pages: Optional[Dict[Any, int]] = None):
        """``run_specs[r]`` is the cache spec of run ``r``, or None.

        ``num_pages`` is the pool size of every paged group unless ``group_pages`` names one for a spec.
        """
        if page_size <= 0:
            raise ValueError(f"page_size must be positive, got {page_size}")
        self.page_size = int(page_size)
        self.run_specs = list(run_specs)
        self.groups: List[CacheGroup] = []
        self.run_group: Dict[int, Tuple[int, int]] = {}   # run -> (group, index within group)
        self.state_runs: Dict[int, Any] = {}
        by_spec: Dict[Any, CacheGroup] = {}
        for run, spec in enumerate(self.run_specs):
            if spec is None:
                continue
            check_spec(spec, run)
            if spec.per_token:
                group = by_spec.get(spec)
                if group is None:
                    pages = (group_pages or {}).get(spec, num_pages)
                    group = CacheGroup(len(self.groups), spec, self.page_size, [], PagePool(pages))
                    by_spec[spec] = group
                    self.groups.append(group)
                self.run_group[run] = (group.index, len(group.runs))
                group.runs.append(run)
            else:
                self.state_runs[run] = spec
        self.slots = StateSlots(max_requests)
        self.requests: Dict[Hashable, _Request] = {}
        self.state: Dict[int, object] = {}  # run -> [slots, *shape] array
        self.max_requests = int(max_requests)
        self._clock = 0     # source of the requests' stamps

    def _tick(self) -> int:
        self._clock += 1
        return self._clock

    # ------------------------------------------------------------------ storage
    def allocate_storage(self, device, dtype) -> None:
        """Create the page and state arrays on ``device``: every spec allocates its own."""
        for g in self.groups:
            g.storage = g.spec.allocate(len(g.runs), g.pool.num_pages, g.page_size, device, dtype)
        for run, spec in self.state_runs.items():
            self.state[run] = spec.allocate(1, self.slots.num_slots, self.page_size, device, dtype)

    def view(self, run: int, writable: bool = True) -> Any:
        """What run ``run`` is handed as its cache in a step (None for a run that keeps nothing)."""
        spec = self.run_specs[run]
        if spec is None:
            return None
        if spec.per_token:
            g, i = self.run_group[run]
            group = self.groups[g]
            return spec.view(group.storage, i, g, group.page_size, writable)
        return spec.view(self.state[run], 0, -1, self.page_size, writable)

    def storage_bytes(self, element_size: int) -> int:
        return sum(len(g.runs) * g.pool.num_pages * g.page_size * g.spec.bytes_per_token(element_size)
                   for g in self.groups)

    # ----------------------------------------------------------------- requests
    def add_request(self, request: Hashable) -> int:
        if request in self.requests:
            raise CacheError(f"request {request!r} is already live")
        slot = self.slots.take(request)
        self.requests[request] = _Request(slot, stamp=self._tick())
        for g in self.groups:
            g.tables[request] = []
        return slot

    def has_request(self, request: Hashable) -> bool:
        return request in self.requests

    def slot_of(self, request: Hashable) -> int:
        return self._req(request).slot

    def computed(self, request: Hashable) -> int:
        return self._req(request).computed

    def reserved(self, request: Hashable) -> int:
        return self._req(request).reserved

    def tables_stamp(self, request: Hashable) -> int:
        """A number that changes whenever a block table of the request changes (a page more, pages given back below
        a window) and that no other request, before or after, has had: who copies the tables elsewhere can tell by
        it whether the copy still holds."""
        return self._req(request).stamp

    def _req(self, request: Hashable) -> _Request:
        try:
            return self.requests[request]
        except KeyError:
            raise CacheError(f"request {request!r} is not live") from None

    def pages_needed(self, request: Hashable, length: int) -> List[int]:
        """Per group, how many more pages the request needs to hold ``length`` tokens."""
        self._req(request)
        return [max(0, g.pages_for(length) - len(g.tables[request])) for g in self.groups]

    def pages_needed_new(self, length: int) -> List[int]:
        """Per group, the pages a request not yet admitted needs for its first ``length`` tokens."""
        return [g.pages_for(length) for g in self.groups]

    def can_reserve(self, request: Optional[Hashable], length: int, spare: Optional[List[int]] = None) -> bool:
        live = self.requests.get(request) if request is not None else None
        if live is not None and length <= live.capacity:
            return True      # the pages it has hold that many tokens
        need = self.pages_needed(request, length) if request in self.requests else self.pages_needed_new(length)
        free = spare if spare is not None else [g.pool.num_free for g in self.groups]
        return all(n <= f for n, f in zip(need, free))

    def free_pages(self) -> List[int]:
        return [g.pool.num_free for g in self.groups]

    def reserve(self, request: Hashable, length: int) -> None:
        """Make sure pages exist for tokens [0, length) in every group; all or nothing."""
        req = self._req(request)
        if length <= req.capacity:   # the pages it has hold that many tokens
            req.reserved = max(req.reserved, length)
            return
        need = self.pages_needed(request, length)
        for g, n in zip(self.groups, need):
            if n > g.pool.num_free:
                raise OutOfPages(f"request {request!r} needs {n} more pages in group {g.index}, "
                                 f"{g.pool.num_free} of {g.pool.num_pages} are free")
        for g, n in zip(self.groups, need):
            g.tables[request].extend(g.pool.allocate(n))
        req.reserved = max(req.reserved, length)
        req.capacity = min((len(g.tables[request]) * g.page_size for g in self.groups), default=1 << 62)
        req.stamp = self._tick()

    def advance(self, request: Hashable, computed: int) -> None:
        """Tokens [0, computed) are now in the cache; give back pages that a window has passed."""
        req = self._req(request)
        if computed < req.computed:
            raise CacheError(f"request {request!r} cannot go back from {req.computed} to {computed} tokens")
        if computed > req.reserved:
            raise CacheError(f"request {request!r} computed {computed} tokens but pages are reserved for {req.reserved}")
        req.computed = computed
        for g in self.groups:
            if g.window is None:
                continue
            table = g.tables[request]
            dead = min(g.first_needed_token(computed) // g.page_size, len(table))
            gone = [table[i] for i in range(dead) if table[i] >= 0]
            if gone:
                g.pool.release(gone)
                for i in range(dead):
                    table[i] = -1
                req.stamp = self._tick()

    def free_request(self, request: Hashable) -> None:
        """Give back everything the request holds (finish or preemption)."""
        req = self._req(request)
        for g in self.groups:
            table = g.tables.pop(request)
            g.pool.release([p for p in table if p >= 0])
        self.slots.give_back(req.slot)
        del self.requests[request]

    def reset(self) -> None:
        for request in list(self.requests):
            self.free_request(request)

    # ------------------------------------------------------------------- tables
    def table(self, group: int, request: Hashable) -> List[int]:
        self._req(request)
        return self.groups[group].tables[request]

    def check(self) -> None:
        """No page lost, held twice or freed twice; tables and pools agree (used by tests)."""
        for g in self.groups:
            g.pool.check()
            held = [p for table in g.tables.values() for p in table if p >= 0]
            if len(held) != len(set(held)):
                raise PageError(f"group {g.index}: a page is in two block tables")
            if len(held) != g.pool.num_held:
                raise PageError(f"group {g.index}: tables hold {len(held)} pages, the pool says {g.pool.num_held}")
            for p in held:
                if not g.pool.is_held(p):
                    raise PageError(f"group {g.index}: page {p} is in a table but free")
            if set(g.tables) != set(self.requests):
                raise PageError(f"group {g.index}: tables and requests disagree")
