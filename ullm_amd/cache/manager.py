"""The cache manager: pages of keys and values with a block table per request and cache group,
and slots for per-request state of fixed size.  Pure host bookkeeping over integer page ids;
the device pools the ids index are owned by the model runner.

Against the reference (ullm/core/kv_cache.py:326-398, ullm/core/req_state.py:6-75): its "page" is a
single token and all layers share one slot id space; a request's row in fixed arrays is an index
from a pool of ``max_bs``.  Here
  * layers with the same needs (kv heads, head size, window) form a *group* with pages of its own
    and one block table per request;
  * a group with a window gives pages back as soon as the window has passed them;
  * pages are handed out per portion (``reserve``) and a request's progress is recorded after the
    step (``commit``); ``release`` gives everything back;
  * a request *slot* (0 .. max_requests-1) stands for the request's rows of fixed-size state (the step
    function zeroes the rows of every request that steps from its first token).
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Dict, List, Optional, Sequence

import numpy as np

from .pages import PageAllocator, PageError
from .prefix_tree import PrefixTree


@dataclass(frozen=True)
class CacheGroupSpec:
    """Layers that keep rows of the same shape and look back the same distance."""
    num_kv_heads: int
    head_dim: int
    window: int                   # 0 = every earlier key
    layers: tuple                 # the caches of this group, one set of pools each (any hashable names)
    # what a token keeps in each layer's pools: (heads, dim, bytes per value or None = the compute dtype's)
    # per pool; None = one key row and one value row per kv head
    rows: Optional[tuple] = None

    def bytes_per_token(self, itemsize: int) -> int:
        rows = self.rows if self.rows is not None else ((self.num_kv_heads, self.head_dim, None),) * 2
        return sum(heads * dim * (size or itemsize) for heads, dim, size in rows) * len(self.layers)


class CacheFull(RuntimeError):
    """No request slot is free."""


@dataclass
class RequestCache:
    request_id: str
    slot: int
    num_computed: int = 0                         # tokens whose rows are written and committed
    tables: List[List[int]] = field(default_factory=list)   # per group: page id by page index, -1 = none
    first_live: List[int] = field(default_factory=list)     # per group: first page index still held
    released: bool = False

    def pages_held(self, group: int) -> List[int]:
        return [p for p in self.tables[group] if p >= 0]


class CacheManager:
    def __init__(self, groups: Sequence[CacheGroupSpec], num_pages: Sequence[int], page_size: int,
                 max_requests: int, enable_prefix_cache: bool = False):
        if len(groups) != len(num_pages):
            raise ValueError("one page count per cache group is needed")
        if page_size < 1 or (page_size & (page_size - 1)):
            raise ValueError("page_size must be a power of two")
        self.groups = list(groups)
        self.page_size = page_size
        self.max_requests = max_requests
        self.allocators = [PageAllocator(n) for n in num_pages]
        self._free_slots: List[int] = list(range(max_requests - 1, -1, -1))
        # the block tables once more as one int32 matrix per group, row = slot, -1 where a table holds
        # no page: a step gathers its rows from here instead of converting Python lists
        self._rows = [np.full((max_requests, 16), -1, dtype=np.int32) for _ in groups]
        self.requests: Dict[str, RequestCache] = {}
        shareable = all(g.window == 0 for g in groups) and len(groups) > 0
        self.prefix_tree: Optional[PrefixTree] = (
            PrefixTree(page_size, self.allocators) if enable_prefix_cache and shareable else None)

    # ------------------------------------------------------------------ requests and slots
    @property
    def num_free_slots(self) -> int:
        return len(self._free_slots)

    def admit(self, request_id: str, prompt: Optional[Sequence[int]] = None) -> RequestCache:
        """Give the request a slot (and, with prefix sharing on, the pages of the longest cached
        prefix of ``prompt`` that leaves at least one token to compute, as the reference does,
        ullm/core/kv_cache.py:349-356)."""
        if request_id in self.requests:
            raise PageError(f"request {request_id!r} is already admitted")
        if not self._free_slots:
            raise CacheFull("every request slot is taken")
        slot = self._free_slots.pop()
        rc = RequestCache(request_id, slot, 0, [[] for _ in self.groups], [0] * len(self.groups))
        if self.prefix_tree is not None and prompt is not None and len(prompt) > 1:
            matched = self.prefix_tree.match(prompt, len(prompt) - 1)
            for per_group in matched:
                for g, page in enumerate(per_group):
                    rc.tables[g].append(page)
            for g in range(len(self.groups)):
                self._put_row(g, slot, 0, rc.tables[g])
            rc.num_computed = len(matched) * self.page_size
        self.requests[request_id] = rc
        return rc

    def _put_row(self, g: int, slot: int, start: int, pages: Sequence[int]) -> None:
        rows = self._rows[g]
        end = start + len(pages)
        if end > rows.shape[1]:
            wider = np.full((rows.shape[0], max(end, 2 * rows.shape[1])), -1, dtype=np.int32)
            wider[:, :rows.shape[1]] = rows
            self._rows[g] = rows = wider
        rows[slot, start:end] = pages

    def table_rows(self, group: int, slots: Sequence[int], width: int) -> np.ndarray:
        """int32 [len(slots), width]: the block tables of the requests in these slots, -1 where a
        table holds no page."""
        rows = self._rows[group]
        if width <= rows.shape[1]:
            return rows[slots, :width]
        out = np.full((len(slots), width), -1, dtype=np.int32)
        out[:, :rows.shape[1]] = rows[slots]
        return out

    # ------------------------------------------------------------------ pages
    def pages_needed(self, rc: RequestCache, n_new: int) -> List[int]:
        """Pages each group lacks for positions [num_computed, num_computed + n_new)."""
        last = (rc.num_computed + n_new - 1) // self.page_size
        return [max(0, last + 1 - len(t)) for t in rc.tables]

    def can_reserve(self, rc: RequestCache, n_new: int) -> bool:
        return all(need <= a.num_free for need, a in zip(self.pages_needed(rc, n_new), self.allocators))

    def reserve(self, rc: RequestCache, n_new: int) -> bool:
        """Make sure every group holds pages for the next ``n_new`` tokens of the request.
        All or nothing: False (and nothing taken) if any group is short even after evicting
        unreferenced prefix pages."""
        if rc.released:
            raise PageError(f"request {rc.request_id!r} was released")
        if n_new < 1:
            raise ValueError("reserve needs at least one token")
        needs = self.pages_needed(rc, n_new)
        if not any(needs):
            return True
        for g, need in enumerate(needs):
            short = need - self.allocators[g].num_free
            if short > 0 and self.prefix_tree is not None:
                self.prefix_tree.evict(g, short)
            if need > self.allocators[g].num_free:
                return False
        for g, need in enumerate(needs):
            if need:
                pages = self.allocators[g].alloc(need)
                assert pages is not None
                self._put_row(g, rc.slot, len(rc.tables[g]), pages)
                rc.tables[g].extend(pages)
        return True

    def commit(self, rc: RequestCache, n_new: int) -> None:
        """Record that ``n_new`` more tokens are in the cache; windowed groups give back the pages
        no later query can reach: page i is dead once (i+1)*page_size <= num_computed - window + 1."""
        if rc.released:
            raise PageError(f"request {rc.request_id!r} was released")
        P = self.page_size
        for g in range(len(self.groups)):
            if rc.num_computed + n_new > len(rc.tables[g]) * P:
                raise PageError(f"request {rc.request_id!r} computed past its reserved pages")
        rc.num_computed += n_new
        for g, spec in enumerate(self.groups):
            if spec.window > 0:
                dead_upto = (rc.num_computed - spec.window + 1) // P   # pages [first_live, dead_upto) die
                table = rc.tables[g]
                for i in range(rc.first_live[g], min(dead_upto, len(table))):
                    if table[i] >= 0:
                        self.allocators[g].decref(table[i])
                        table[i] = -1
                        self._rows[g][rc.slot, i] = -1
                rc.first_live[g] = max(rc.first_live[g], min(dead_upto, len(table)))

    def release(self, rc: RequestCache, tokens: Optional[Sequence[int]] = None) -> None:
        """The request ends (finished, aborted or preempted): every page loses this holder and the
        slot is free again.  With prefix sharing on and ``tokens`` given, full computed pages are
        offered to the prefix tree first (the reference caches at finish, kv_cache.py:358-398)."""
        if rc.released:
            raise PageError(f"request {rc.request_id!r} released twice")
        if self.prefix_tree is not None and tokens is not None:
            self.prefix_tree.insert(tokens, min(rc.num_computed, len(tokens)), rc.tables)
        for g, table in enumerate(rc.tables):
            for p in table:
                if p >= 0:
                    self.allocators[g].decref(p)
            table.clear()
            self._rows[g][rc.slot] = -1
        rc.released = True
        self._free_slots.append(rc.slot)
        del self.requests[rc.request_id]

    def rewind(self, rc: RequestCache) -> None:
        """Forget the request's cache but keep its slot (recompute from the first token)."""
        for g, table in enumerate(rc.tables):
            for p in table:
                if p >= 0:
                    self.allocators[g].decref(p)
            table.clear()
            self._rows[g][rc.slot] = -1
            rc.first_live[g] = 0
        rc.num_computed = 0

    # ------------------------------------------------------------------ figures and checks
    def num_free_pages(self, group: int = 0) -> int:
        return self.allocators[group].num_free

    def max_table_len(self, rcs: Sequence[RequestCache], group: int) -> int:
        return max((len(rc.tables[group]) for rc in rcs), default=0)

    def check(self) -> None:
        """No page lost, held twice by unrelated holders, or freed twice; slots conserved."""
        for g, alloc in enumerate(self.allocators):
            alloc.check()
            holders = [0] * alloc.num_pages
            for rc in self.requests.values():
                seen = set()
                for p in rc.tables[g]:
                    if p < 0:
                        continue
                    if p in seen:
                        raise PageError(f"page {p} twice in the table of {rc.request_id!r}")
                    seen.add(p)
                    holders[p] += 1
            tree_pages = set()
            if self.prefix_tree is not None:
                for p in self.prefix_tree.pages_held(g):
                    if p in tree_pages:
                        raise PageError(f"page {p} twice in the prefix tree")
                    tree_pages.add(p)
                    holders[p] += 1
            for p in range(alloc.num_pages):
                if holders[p] != alloc.refcount(p):
                    raise PageError(f"group {g} page {p}: {holders[p]} holders found, count says {alloc.refcount(p)}")
                if holders[p] > 1 and p not in tree_pages:
                    raise PageError(f"group {g} page {p} is in {holders[p]} block tables without a shared prefix")
        for g in range(len(self.groups)):
            held = np.full_like(self._rows[g], -1)
            for rc in self.requests.values():
                held[rc.slot, :len(rc.tables[g])] = rc.tables[g]
            if not np.array_equal(held, self._rows[g]):
                raise PageError(f"group {g}: the table matrix differs from the requests' block tables")
        slots = [rc.slot for rc in self.requests.values()]
        if len(set(slots)) != len(slots) or set(slots) & set(self._free_slots):
            raise PageError("a request slot is held twice")
        if len(slots) + len(self._free_slots) != self.max_requests:
            raise PageError("a request slot was lost")
