"""Prefix sharing at page granularity.

The reference keeps a compressed radix tree keyed by single tokens whose values are one-token
slots, with per-node reference counts walked up to the root and eviction of unreferenced leaves
by access time (ullm/core/kv_cache.py:137-323).  With pages of several tokens only whole pages
can be shared, so an edge here is one full page of token ids and a node owns one page per cache
group.  Who may free a page is decided by the page's own reference count (the tree is one holder
among the requests), which removes the reference's hazards around preemption and duplicate
prefixes (kv_cache.py:378 frees duplicates only when a prefix was matched at admission;
ullm/core/scheduler.py:160-183 frees tree-owned slots on preemption).
"""
from __future__ import annotations

import heapq
import itertools
from typing import Dict, List, Optional, Sequence, Tuple

from .pages import PageAllocator


class _Node:
    __slots__ = ("key", "pages", "children", "parent", "stamp")

    def __init__(self, key: Tuple[int, ...], pages: List[int], parent: Optional["_Node"]):
        self.key = key
        self.pages = pages              # one page id per cache group
        self.children: Dict[Tuple[int, ...], "_Node"] = {}
        self.parent = parent
        self.stamp = 0


class PrefixTree:
    def __init__(self, page_size: int, allocators: Sequence[PageAllocator]):
        self.page_size = page_size
        self.allocators = list(allocators)
        self.root = _Node((), [], None)
        self._clock = itertools.count(1)
        self.num_nodes = 0

    def _keys(self, tokens: Sequence[int], limit: int):
        P = self.page_size
        for i in range(limit // P):
            yield tuple(int(t) for t in tokens[i * P:(i + 1) * P])

    def match(self, tokens: Sequence[int], limit: int) -> List[List[int]]:
        """Pages of the longest cached prefix of ``tokens[:limit]`` made of whole pages:
        a list (one entry per matched page) of per-group page ids.  Every returned page gets
        one more holder (the caller's block table)."""
        node = self.root
        out: List[List[int]] = []
        for key in self._keys(tokens, limit):
            child = node.children.get(key)
            if child is None:
                break
            child.stamp = next(self._clock)
            for alloc, page in zip(self.allocators, child.pages):
                alloc.incref(page)
            out.append(list(child.pages))
            node = child
        return out

    def insert(self, tokens: Sequence[int], num_computed: int, tables: Sequence[Sequence[int]]) -> int:
        """Offer the full pages of ``tokens[:num_computed]`` held in ``tables`` (per group, page id by
        page index).  Pages of new nodes get the tree as one more holder.  Where the tree already has
        a node for the same tokens it keeps its own page.  Returns the number of nodes added."""
        node = self.root
        added = 0
        for i, key in enumerate(self._keys(tokens, num_computed)):
            child = node.children.get(key)
            if child is None:
                pages = [int(t[i]) for t in tables]
                if any(p < 0 for p in pages):
                    break
                for alloc, page in zip(self.allocators, pages):
                    alloc.incref(page)
                child = _Node(key, pages, node)
                node.children[key] = child
                self.num_nodes += 1
                added += 1
            child.stamp = next(self._clock)
            node = child
        return added

    def evict(self, group: int, need: int) -> int:
        """Drop least recently used leaves that only the tree still holds until ``need`` pages of
        ``group`` came free (or nothing evictable is left).  Returns pages freed in that group."""
        heap = [(n.stamp, id(n), n) for n in self._leaves()]
        heapq.heapify(heap)
        freed = 0
        while heap and freed < need:
            _, _, node = heapq.heappop(heap)
            if node is self.root or node.children:
                continue
            if any(a.refcount(p) != 1 for a, p in zip(self.allocators, node.pages)):
                continue  # a request still reads it
            for g, (alloc, page) in enumerate(zip(self.allocators, node.pages)):
                if alloc.decref(page) and g == group:
                    freed += 1
            parent = node.parent
            del parent.children[node.key]
            self.num_nodes -= 1
            if parent is not self.root and not parent.children:
                heapq.heappush(heap, (parent.stamp, id(parent), parent))
        return freed

    def _leaves(self):
        stack = [self.root]
        while stack:
            n = stack.pop()
            if not n.children and n is not self.root:
                yield n
            stack.extend(n.children.values())

    def pages_held(self, group: int) -> List[int]:
        out = []
        stack = list(self.root.children.values())
        while stack:
            n = stack.pop()
            out.append(n.pages[group])
            stack.extend(n.children.values())
        return out

    def clear(self) -> None:
        stack = list(self.root.children.values())
        while stack:
            n = stack.pop()
            for alloc, page in zip(self.allocators, n.pages):
                alloc.decref(page)
            stack.extend(n.children.values())
        self.root.children.clear()
        self.num_nodes = 0
