"""First-come-first-served continuous batching under a token budget.

Reference: ullm/core/scheduler.py:15-225.  The reference schedules either whole prompts or one
token per running request, has no token budget, and only its decode path survives running out of
cache (scheduler.py:114-128); admission lets the allocation error escape.  Here every step is
  1. one token for every running request that is decoding,
  2. a portion min(rest, budget left, max_prefill_chunk) for running requests still in their prompt,
  3. admission of waiting requests in arrival order, each with a first portion, while a request
     slot, budget and pages last; the first that does not fit stops admission (no overtaking).
Pages are reserved per portion.  When pages run out for a running request the youngest running
request is preempted: its pages are given back, it returns to the front of the waiting queue and is
later recomputed from all its tokens, prompt and generated (the reference's policy,
scheduler.py:121-124,169-183).  If the request that cannot grow is the only one left, it ends with
reason LENGTH: it already holds everything the pool can hold.  A prompt that needs more pages than
the pool has is refused when it is added.
"""
from __future__ import annotations

from collections import deque
from typing import Deque, Dict, List, Optional

from ..cache.manager import CacheManager
from .request import FinishReason, Request, RequestStatus, Scheduled


class Scheduler:
    def __init__(self, cache: CacheManager, max_num_batched_tokens: int, max_prefill_chunk: int, max_bs: int):
        self.cache = cache
        self.token_budget = max_num_batched_tokens
        self.max_prefill_chunk = max_prefill_chunk
        self.max_bs = min(max_bs, cache.max_requests)
        self.waiting: Deque[Request] = deque()
        self.running: List[Request] = []              # in admission order: oldest first
        self.requests: Dict[str, Request] = {}
        self.finished_by_scheduler: List[Request] = []   # ended because the pool cannot hold more
        self.num_preemptions = 0

    # ------------------------------------------------------------------ queue
    def add(self, req: Request) -> None:
        if req.request_id in self.requests:
            raise ValueError(f"request id {req.request_id!r} is already in use")
        P = self.cache.page_size
        need = -(-(req.num_tokens) // P)
        smallest = min(a.num_pages for a in self.cache.allocators) if self.cache.allocators else need
        if need > smallest:
            raise ValueError(f"request {req.request_id!r}: a prompt of {req.num_tokens} tokens needs {need} "
                             f"pages but the cache has {smallest}")
        req.status = RequestStatus.WAITING
        self.waiting.append(req)
        self.requests[req.request_id] = req

    def has_unfinished(self) -> bool:
        return bool(self.waiting or self.running)

    # ------------------------------------------------------------------ scheduling
    def schedule(self) -> List[Scheduled]:
        budget = self.token_budget
        out: List[Scheduled] = []
        decoding = [r for r in self.running if r.num_tokens - r.num_computed == 1]
        prefilling = [r for r in self.running if r.num_tokens - r.num_computed > 1]
        for req in decoding + prefilling:
            if req.status is not RequestStatus.RUNNING or budget <= 0:
                continue   # preempted earlier in this very call, or nothing left to give
            rest = req.num_tokens - req.num_computed
            n = min(rest, budget, self.max_prefill_chunk) if rest > 1 else 1
            if self._reserve_or_preempt(req, n, out):
                out.append(Scheduled(req, req.num_computed, n))
                budget -= n
        while self.waiting and budget > 0 and len(self.running) < self.max_bs and self.cache.num_free_slots > 0:
            req = self.waiting[0]
            rc = self.cache.admit(req.request_id, req.token_ids)
            rest = req.num_tokens - rc.num_computed
            n = min(rest, budget, self.max_prefill_chunk)
            if not self.cache.reserve(rc, n):
                self.cache.release(rc)
                break
            self.waiting.popleft()
            req.cache = rc
            req.status = RequestStatus.RUNNING
            self.running.append(req)
            out.append(Scheduled(req, rc.num_computed, n))
            budget -= n
        return out

    def _reserve_or_preempt(self, req: Request, n: int, scheduled: List[Scheduled]) -> bool:
        while not self.cache.reserve(req.cache, n):
            victim = self.running[-1]
            if victim is req:
                if len(self.running) == 1:
                    # alone and still short: it holds all the pool can give
                    self._finish_for_capacity(req)
                else:
                    self.preempt(req)
                return False
            for i, s in enumerate(scheduled):
                if s.request is victim:
                    del scheduled[i]
                    break
            self.preempt(victim)
        return True

    def preempt(self, req: Request) -> None:
        """Back to the front of the waiting queue without any cache (reference: scheduler.py:169-183)."""
        if req.status is not RequestStatus.RUNNING:
            return
        self.running.remove(req)
        self.cache.release(req.cache)
        req.cache = None
        req.status = RequestStatus.WAITING
        req.num_preemptions += 1
        self.num_preemptions += 1
        self.waiting.appendleft(req)

    def _finish_for_capacity(self, req: Request) -> None:
        req.finish_reason = FinishReason.LENGTH
        self.finish(req)
        self.finished_by_scheduler.append(req)

    # ------------------------------------------------------------------ after the step
    def append_token(self, req: Request, token: int) -> None:
        if req.status is RequestStatus.RUNNING:
            req.token_ids.append(int(token))

    def finish(self, req: Request) -> None:
        """Ends a request in any state: finished, aborted (reference: scheduler.py:204-222)."""
        if req.status is RequestStatus.FINISHED:
            return
        if req.status is RequestStatus.WAITING:
            self.waiting.remove(req)
        elif req.status is RequestStatus.RUNNING:
            self.running.remove(req)
            self.cache.release(req.cache, tokens=req.token_ids)
            req.cache = None
        req.status = RequestStatus.FINISHED
        self.requests.pop(req.request_id, None)
