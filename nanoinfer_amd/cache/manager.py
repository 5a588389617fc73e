"""The cache manager: pages of keys and values with a block table per request, and slots for
per-request state of fixed size.

The reference has one pool geometry for all layers and one table per sequence
(src/engine/kv_cache_manager.cpp:42-220, src/engine/block_table.cpp:22-230).  Here the caches of
a model are put into *groups* by what they need: caches that keep all keys of the same geometry
share one group, caches that keep a window of n keys another.  A group has page ids and block
tables of its own; every cache in it has its own key and value pool, indexed by the group's page
ids.  Pages are taken when tokens are reserved, handed back when a request is released, and, in
a windowed group, as soon as the window has moved past them; they are handed out again LIFO.

Beside the pages sit :class:`StateSlots`: one slot index per live request, valid in every state
tensor ``[slots, *shape]`` that a cache asked for.  Slots are given and taken back with the
request even when no cache of the model holds state.

All bookkeeping is host-only and needs no GPU; pools are allocated only when a device is given.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Dict, Hashable, List, Optional, Tuple

import torch

from ..parts.base import CacheNeed, KVNeed, StateNeed
from .block_manager import BlockManager, OutOfPages


class CacheError(RuntimeError):
    pass


class StateSlots:
    """Slot indices for per-request state: a free list, request -> slot."""

    def __init__(self, num_slots: int):
        self.num_slots = int(num_slots)
        self._free = list(range(self.num_slots - 1, -1, -1))
        self._of: Dict[Hashable, int] = {}

    @property
    def num_free(self) -> int:
        return len(self._free)

    def take(self, request: Hashable) -> int:
        if request in self._of:
            raise CacheError(f"request {request!r} already holds state slot {self._of[request]}")
        if not self._free:
            raise OutOfPages(f"all {self.num_slots} state slots are taken")
        s = self._free.pop()
        self._of[request] = s
        return s

    def give_back(self, request: Hashable) -> int:
        if request not in self._of:
            raise CacheError(f"request {request!r} holds no state slot")
        s = self._of.pop(request)
        self._free.append(s)
        return s

    def slot(self, request: Hashable) -> int:
        return self._of[request]

    def __contains__(self, request: Hashable) -> bool:
        return request in self._of


@dataclass
class KVGroup:
    """Caches with one need: geometry (kv heads, head size) and reach (all keys or a window)."""

    need: KVNeed
    cache_ids: List[int]
    page_size: int
    pages: BlockManager
    tables: Dict[Hashable, List[int]] = field(default_factory=dict)   # logical page -> page id, -1 once given back
    kpools: Dict[int, torch.Tensor] = field(default_factory=dict)     # cache id -> [pages, kv_heads, page_size, hd]
    vpools: Dict[int, torch.Tensor] = field(default_factory=dict)

    def first_needed_page(self, next_position: int) -> int:
        """Logical index of the first page that a query at ``next_position`` can still read."""
        if self.need.window is None:
            return 0
        first_key = max(0, next_position + 1 - self.need.window)
        return first_key // self.page_size


class ReservationPlan:
    """Reservations that are to be made together, collected one by one: ``fits`` says whether one
    more ``(request, total_tokens)`` can be reserved beside those already added, in time that does
    not grow with their number (a scheduler asks once per request and step).  Pages that are
    freed while the plan is filled only make more fit; the plan reserves nothing itself."""

    def __init__(self, cache: "KVCacheManager"):
        self.cache = cache
        self.new_pages = [0] * len(cache.groups)
        self.new_requests = 0
        self.wanted: List[Tuple[Hashable, int]] = []

    def _needs(self, request: Hashable, total_tokens: int):
        c = self.cache
        return [c._new_pages_needed(g, request, total_tokens) for g in c.groups]

    def fits(self, request: Hashable, total_tokens: int) -> bool:
        c = self.cache
        if request not in c._tokens and self.new_requests + 1 > c.slots.num_free:
            return False
        return all(g.pages.can_allocate(have + n)
                   for g, have, n in zip(c.groups, self.new_pages, self._needs(request, total_tokens)))

    def free_after(self, request: Hashable, total_tokens: int) -> int:
        """Pages that the fullest group would still have free with this reservation beside those added."""
        c = self.cache
        return min((g.pages.num_free - have - n
                    for g, have, n in zip(c.groups, self.new_pages, self._needs(request, total_tokens))),
                   default=c.num_pages)

    def add(self, request: Hashable, total_tokens: int) -> None:
        if request not in self.cache._tokens:
            self.new_requests += 1
        for i, n in enumerate(self._needs(request, total_tokens)):
            self.new_pages[i] += n
        self.wanted.append((request, total_tokens))


class KVCacheManager:
    """Pages and state slots for the caches of one model.

    ``needs[c]`` is what cache ``c`` wants.  ``num_pages`` is the size of the pool of a group that
    keeps all keys, in pages of ``page_size`` tokens.  A group that keeps a window of n keys never
    holds more of a request than its window and the tokens of one step: when ``max_step_tokens``
    (the most tokens one request brings to one step) is given, such a group's pool is only as
    large as ``max_requests`` requests can fill, and no larger than ``num_pages``; without it every
    group gets ``num_pages``.  ``device=None`` keeps the books without allocating pools.
    ``scatter_pages`` hands page ids out in a fixed pseudo-random order (see :class:`BlockManager`).
    """

    def __init__(self, needs: Dict[int, CacheNeed], page_size: int, num_pages: int, max_requests: int,
                 dtype: torch.dtype = torch.float32, device: Optional[torch.device] = None,
                 max_step_tokens: Optional[int] = None, scatter_pages: bool = False):
        if page_size < 1:
            raise ValueError(f"page_size must be at least 1, got {page_size}")
        self.page_size = int(page_size)
        self.num_pages = int(num_pages)
        self.max_step_tokens = None if max_step_tokens is None else int(max_step_tokens)
        self.dtype = dtype
        self.device = device
        self.groups: List[KVGroup] = []
        self.group_of_cache: Dict[int, int] = {}
        self.state_needs: Dict[int, StateNeed] = {}
        self.state: Dict[int, torch.Tensor] = {}
        by_need: Dict[KVNeed, int] = {}
        for cid in sorted(needs):
            need = needs[cid]
            if need.kv is not None:
                gi = by_need.get(need.kv)
                if gi is None:
                    gi = len(self.groups)
                    by_need[need.kv] = gi
                    self.groups.append(KVGroup(need.kv, [], self.page_size, BlockManager(self.pages_of_group(need.kv, max_requests), scatter=scatter_pages)))
                self.groups[gi].cache_ids.append(cid)
                self.group_of_cache[cid] = gi
            if need.state is not None:
                self.state_needs[cid] = need.state
        self.slots = StateSlots(max_requests)
        self._tokens: Dict[Hashable, int] = {}
        if device is not None:
            for g in self.groups:
                shape = (g.pages.num_pages, g.need.kv_heads, self.page_size, g.need.head_dim)
                for cid in g.cache_ids:
                    g.kpools[cid] = torch.zeros(shape, dtype=dtype, device=device)
                    g.vpools[cid] = torch.zeros(shape, dtype=dtype, device=device)
            for cid, sn in self.state_needs.items():
                self.state[cid] = torch.zeros((max_requests,) + tuple(sn.shape), dtype=sn.dtype, device=device)

    def pages_of_group(self, need: KVNeed, max_requests: int) -> int:
        """Pages in the pool of a group with this need.  A windowed group holds of one request at most
        the pages that its window and one step's tokens touch: before a step the keys of the window,
        during it the step's tokens as well, and a run of n keys touches at most
        ``ceil(n / page_size) + 1`` pages."""
        if need.window is None or self.max_step_tokens is None:
            return self.num_pages
        per_request = -(-(int(need.window) + self.max_step_tokens) // self.page_size) + 1
        return min(self.num_pages, int(max_requests) * per_request)

    # ---------------------------------------------------------------- queries
    def has(self, request: Hashable) -> bool:
        return request in self._tokens

    def num_tokens(self, request: Hashable) -> int:
        """Tokens reserved for the request so far (src/engine/kv_cache_manager.cpp:120,176)."""
        return self._tokens[request]

    def live_requests(self) -> List[Hashable]:
        return list(self._tokens)

    def state_slot(self, request: Hashable) -> int:
        return self.slots.slot(request)

    def block_table(self, group: int, request: Hashable) -> List[int]:
        return self.groups[group].tables[request]

    def free_pages(self, group: int = 0) -> int:
        return self.groups[group].pages.num_free if self.groups else 0

    def min_free_pages(self) -> int:
        return min((g.pages.num_free for g in self.groups), default=self.num_pages)

    def pool_bytes(self) -> int:
        """Bytes of all key and value pools together."""
        el = torch.empty(0, dtype=self.dtype).element_size()
        return sum(2 * len(g.cache_ids) * g.pages.num_pages * g.need.kv_heads * self.page_size * g.need.head_dim * el
                   for g in self.groups)

    @staticmethod
    def pages_for_bytes(needs: Dict[int, CacheNeed], page_size: int, budget_bytes: int, dtype: torch.dtype) -> int:
        """The largest ``num_pages`` whose pools fit ``budget_bytes`` when every cache of ``needs`` that
        holds keys and values gets that many pages (windowed groups may then be given fewer)."""
        el = torch.empty(0, dtype=dtype).element_size()
        per_page = sum(2 * n.kv.kv_heads * page_size * n.kv.head_dim * el for n in needs.values() if n.kv is not None)
        return int(budget_bytes // per_page) if per_page else 0

    def utilization(self) -> float:
        return max((g.pages.utilization() for g in self.groups), default=0.0)

    def pages_for(self, tokens: int) -> int:
        """``ceil(tokens / page_size)`` (include/nanoinfer/engine/kv_cache_manager.h:111-113)."""
        return (tokens + self.page_size - 1) // self.page_size

    def _new_pages_needed(self, g: KVGroup, request: Hashable, total: int) -> int:
        have = len(g.tables.get(request, ()))
        return max(0, self.pages_for(total) - have)

    def can_reserve(self, request: Hashable, total_tokens: int) -> bool:
        if request not in self._tokens and self.slots.num_free == 0:
            return False
        return all(g.pages.can_allocate(self._new_pages_needed(g, request, total_tokens)) for g in self.groups)

    def can_reserve_all(self, wanted) -> bool:
        """Whether all ``(request, total_tokens)`` pairs can be reserved together."""
        wanted = list(wanted)
        new_requests = sum(1 for r, _ in wanted if r not in self._tokens)
        if new_requests > self.slots.num_free:
            return False
        return all(g.pages.can_allocate(sum(self._new_pages_needed(g, r, t) for r, t in wanted)) for g in self.groups)

    def plan(self) -> "ReservationPlan":
        """An empty plan of reservations to be made together (what a scheduler fills for one step)."""
        return ReservationPlan(self)

    def max_tokens_per_request(self) -> int:
        """The longest request the pools can ever hold: it then holds every page of a group that keeps
        all keys.  (A model whose groups all keep windows is bounded by its positions alone.)"""
        full = [g.pages.num_pages for g in self.groups if g.need.window is None]
        if full:
            return min(full) * self.page_size
        return self.num_pages * self.page_size if not self.groups else 1 << 60

    # ---------------------------------------------------------------- changes
    def reserve(self, request: Hashable, total_tokens: int) -> bool:
        """Make room for the request's tokens ``0..total_tokens-1`` in every group; a request seen
        for the first time also gets its state slot.  All or nothing: ``False`` leaves everything
        as it was (src/engine/kv_cache_manager.cpp:94-183, all-or-nothing as block_manager.cpp:66-70)."""
        known = request in self._tokens
        if known and total_tokens < self._tokens[request]:
            raise CacheError(f"request {request!r} holds {self._tokens[request]} tokens, cannot shrink to {total_tokens}")
        if not self.can_reserve(request, total_tokens):
            return False
        if not known:
            slot = self.slots.take(request)
            for cid, t in self.state.items():
                t[slot].zero_()
            for g in self.groups:
                g.tables[request] = []
        for g in self.groups:
            g.tables[request].extend(g.pages.allocate(self._new_pages_needed(g, request, total_tokens)))
        self._tokens[request] = total_tokens
        return True

    def reserve_all(self, wanted) -> bool:
        """:meth:`reserve` for several ``(request, total_tokens)`` pairs at once, all or nothing,
        with one pass over the books (the common case of a decode step: no request needs a page)."""
        wanted = list(wanted)
        tokens = self._tokens
        page = self.page_size
        new = [r for r, _ in wanted if r not in tokens]
        if len(new) > self.slots.num_free:
            return False
        needs = []
        for g in self.groups:
            tables = g.tables
            per = []
            total_new = 0
            for r, t in wanted:
                held = tokens.get(r)
                if held is not None and t < held:
                    raise CacheError(f"request {r!r} holds {held} tokens, cannot shrink to {t}")
                n = (t + page - 1) // page - len(tables.get(r, ()))
                if n > 0:
                    per.append((r, n))
                    total_new += n
            if not g.pages.can_allocate(total_new):
                return False
            needs.append(per)
        for r in new:
            slot = self.slots.take(r)
            for cid, t in self.state.items():
                t[slot].zero_()
            for g in self.groups:
                g.tables[r] = []
        for g, per in zip(self.groups, needs):
            for r, n in per:
                g.tables[r].extend(g.pages.allocate(n))
        for r, t in wanted:
            tokens[r] = t
        return True

    def release_passed(self, request: Hashable, next_position: int) -> int:
        """Give back the pages of windowed groups that no query at ``next_position`` or later can
        read.  Their table entries become -1.  Returns how many pages were freed."""
        freed = 0
        for g in self.groups:
            if g.need.window is None:
                continue
            table = g.tables[request]
            upto = min(len(table), g.first_needed_page(next_position))
            gone = [table[i] for i in range(upto) if table[i] >= 0]
            if gone:
                g.pages.free(gone)
                for i in range(upto):
                    table[i] = -1
                freed += len(gone)
        return freed

    def release(self, request: Hashable) -> None:
        """The request is over: all its pages and its state slot go back
        (src/engine/kv_cache_manager.cpp:186-220)."""
        if request not in self._tokens:
            raise CacheError(f"request {request!r} holds nothing")
        for g in self.groups:
            g.pages.free([p for p in g.tables.pop(request) if p >= 0])
        self.slots.give_back(request)
        del self._tokens[request]

    def reset(self) -> None:
        for r in list(self._tokens):
            self.release(r)

    # ---------------------------------------------------------------- invariants (used by tests)
    def check(self) -> None:
        """Every page is free or held by exactly one request; counts add up."""
        for gi, g in enumerate(self.groups):
            held = [p for t in g.tables.values() for p in t if p >= 0]
            if len(held) != len(set(held)):
                raise CacheError(f"group {gi}: a page is held twice")
            if len(held) != g.pages.num_taken:
                raise CacheError(f"group {gi}: {len(held)} pages in tables, {g.pages.num_taken} marked taken")
            for p in held:
                if not g.pages.is_taken(p):
                    raise CacheError(f"group {gi}: page {p} is in a table but marked free")
            if set(g.tables) != set(self._tokens):
                raise CacheError(f"group {gi}: tables and requests differ")
        if self.slots.num_free + len(self._tokens) != self.slots.num_slots:
            raise CacheError("state slots do not add up")
