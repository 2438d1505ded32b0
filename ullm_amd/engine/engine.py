"""The engine: scheduler + step function + sampler, one process, one GPU.

Reference: ullm/core/engine.py:24-238 (add_sequence, abort_sequence, step = schedule -> execute ->
update_from_output, finish rules) with ullm/core/model_runner.py:123-183,233-255 folded in (model
load, cache sizing from free memory).
"""
from __future__ import annotations

import logging
from dataclasses import dataclass, field
from typing import Dict, List, Optional, Sequence

import torch

from ..config.engine_config import EngineConfig
from ..sampling import Sampler, SamplingParams
from .loading import load_model, random_model
from .request import EngineStepResult, FinishReason, Request, RequestStatus, Scheduled
from .runner import UNKNOWN_TOKEN, ModelRunner, PreparedStep, StepEntry
from .scheduler import Scheduler

logger = logging.getLogger("ullm_amd")


def pages_from_memory(model, env, page_size: int, utilization: float, context_len: int, max_bs: int) -> List[int]:
    """Pages per cache group from free device memory (reference: bytes per token =
    layers * kv_heads * head_dim * 2 * itemsize; tokens = free * utilization // that,
    ullm/core/model_runner.py:233-255), capped at what max_bs requests of context_len can use."""
    groups, _, _ = model.cache_layout()
    if not groups:
        return []
    free, _ = torch.cuda.mem_get_info(env.device)
    itemsize = torch.empty((), dtype=env.dtype).element_size()
    per_token = sum(g.bytes_per_token(itemsize) for g in groups)
    tokens = int(free * utilization) // max(1, per_token)
    cap = max_bs * (-(-context_len // page_size))
    pages = min(tokens // page_size, cap)
    if pages < 1:
        raise RuntimeError("no device memory left for the cache after loading the model")
    return [pages] * len(groups)


@dataclass
class _Plan:
    """A scheduled step with its host work done."""
    scheduled: List[Scheduled]
    early_results: List[EngineStepResult]                 # requests the scheduler itself ended
    sampling: List[Scheduled] = field(default_factory=list)
    sample_positions: List[int] = field(default_factory=list)   # index each new token takes in its request
    prepared: Optional[PreparedStep] = None
    sampler_staged: Optional[torch.Tensor] = None         # the sampling parameters in pinned memory


class Engine:
    def __init__(self, config: EngineConfig, model=None, env=None, model_config=None):
        """``model``/``env``/``model_config`` may be handed in already built (random weights on the
        device, tests); otherwise the folder ``config.model`` is loaded."""
        self.config = config
        logging.basicConfig(level=getattr(logging, config.log_level.upper(), logging.INFO))
        if model is None and config.random_weights is not None:
            model_config, model, env = random_model(config.random_weights, config.dtype, config.device, config.context_len)
        elif model is None:
            model_config, model, env = load_model(config.model, config.dtype, config.device, config.context_len)
        self.model_config, self.model, self.env = model_config, model, env
        if config.num_pages is not None:
            groups, _, _ = model.cache_layout()
            num_pages = [config.num_pages] * len(groups)
        else:
            num_pages = pages_from_memory(model, env, config.page_size, config.gpu_memory_utilization,
                                          config.context_len, config.max_bs)
        self.runner = ModelRunner(model, env, config.page_size, num_pages, config.max_bs,
                                  enable_prefix_cache=config.enable_prefix_cache,
                                  use_graphs=not config.enforce_eager)
        self.scheduler = Scheduler(self.runner.cache, config.max_num_batched_tokens, config.max_prefill_chunk,
                                   config.max_bs)
        self.sampler = Sampler(env.device)
        # the sampled ids of the step that ran last, on the device: the next step takes late token ids from
        # here; each step's ids also go to pinned host memory (two buffers in turn) right behind its sampling
        self._sampled_dev = torch.zeros(max(1, config.max_bs), dtype=torch.int32, device=env.device)
        self.runner.feed_source = self._sampled_dev
        pin = env.device.type == "cuda"
        self._sampled_host = [torch.zeros(max(1, config.max_bs), dtype=torch.int32, pin_memory=pin) for _ in range(2)]
        self._sampled_turn = 0
        self._arrivals = 0
        self._next: Optional[_Plan] = None   # the step after the one that ran last, scheduled and packed ahead
        self._inflight = None                # (plan, sampled ids on the device) of a step that is running
        self.on_logits = None      # optional callable(scheduled that sample, float32 logits): for inspection
        logger.info("cache: %s pages of %d tokens per group, %.2f GiB", num_pages, config.page_size,
                    self.runner.cache_bytes() / 2 ** 30)

    # ------------------------------------------------------------------ requests
    def add_request(self, request_id: str, prompt_token_ids: Sequence[int], params: SamplingParams) -> Request:
        """Reference: ullm/core/engine.py:72-90 (a prompt longer than context_len keeps its last
        context_len tokens, engine.py:81-82)."""
        prompt = [int(t) for t in prompt_token_ids]
        if not prompt:
            raise ValueError("a request needs at least one prompt token")
        if len(prompt) > self.config.context_len:
            prompt = prompt[-self.config.context_len:]
        for t in prompt:
            if not (0 <= t < self.runner.vocab_size):
                raise ValueError(f"prompt token id {t} outside [0, {self.runner.vocab_size})")
        if params.eos_token_id == -1:
            # config.json may name several stop ids: the first becomes the request's eos_token_id (the
            # reference knows one, ullm/llm.py:93-94), the others join its stop_token_ids
            ids = tuple(getattr(self.model_config, "eos_token_ids", ()) or ())
            if ids:
                params.eos_token_id = ids[0]
                params.stop_token_ids = list(params.stop_token_ids) + [t for t in ids[1:] if t not in params.stop_token_ids]
        order = self._arrivals
        self._arrivals += 1
        seed = params.seed if params.seed is not None else (self.config.seed * 1000003 + order)
        req = Request(request_id, prompt, len(prompt), params, seed, order)
        self.scheduler.add(req)
        return req

    def abort_request(self, request_id: str) -> None:
        req = self.scheduler.requests.get(request_id)
        if req is not None:
            self.scheduler.finish(req)
            self._drop_from_next(req)

    def drain(self) -> None:
        """Wait for a step that is still running on the device (its results are dropped)."""
        if self._inflight is not None:
            _, handle = self._inflight
            self._inflight = None
            if handle is not None:
                self._read_sampled(handle)
        if self.env.device.type == "cuda":
            torch.cuda.synchronize(self.env.device)

    def has_unfinished_requests(self) -> bool:
        """True while a request waits or runs, or a prepared step still has an ending to report."""
        return self.scheduler.has_unfinished() or (self._next is not None and bool(self._next.early_results))

    # ------------------------------------------------------------------ one step
    def step(self) -> List[EngineStepResult]:
        """One engine step: the scheduled batch runs, its requests that reached the end of their
        tokens get one new token each; returns what happened to them.

        The device works asynchronously, and the host uses that (reference: the overlap of scheduling
        and execution, docs/async_scheduling.md; ``disable_async_scheduling`` switches it off).
        While a step's kernels run, the next step is scheduled, packed and queued behind it: what it
        depends on is known without the tokens that are still being sampled (counts decide who
        continues; the ids stay on the device, where the next step picks them up from the sampler's
        output, as the reference's device-resident last token does, docs/async_scheduling.md:13).
        Only then does the host wait for this step's tokens and file them.  A request that ends on
        its stop token (the one surprise) has one more token computed in the step already queued;
        that step's result for it is dropped.  So a call returns the results of one step while the
        next one is already running, and the device never waits for the host."""
        if self.config.disable_async_scheduling:
            return self._step_in_turn()
        if self._inflight is None:
            plan, self._next = self._next, None
            if plan is None or not (plan.scheduled or plan.early_results):
                plan = self._make_plan()      # nothing was prepared (or nothing was there to prepare then)
            if not plan.scheduled:
                return plan.early_results
            self._inflight = self._launch(plan)
        plan, sampled = self._inflight
        self._inflight = None
        results = plan.early_results
        sampling = plan.sampling
        if sampled is None:                               # prompt portions only: nothing to wait for
            nxt = self._make_plan()
            if nxt.scheduled:
                self._inflight = self._launch(nxt)
            elif nxt.early_results:
                self._next = nxt
            return results
        # while the device works: who ends by length, and the next step
        ended: Dict[int, FinishReason] = {}
        filed = []                                        # index of each new token in its request (None: aborted meanwhile)
        for i, s in enumerate(sampling):
            req = s.request
            if req.status is not RequestStatus.RUNNING:
                filed.append(None)
                continue
            filed.append(req.num_tokens)
            self.scheduler.append_token(req, UNKNOWN_TOKEN)
            reason = self._ends_by_length(req)
            if reason is not None:
                ended[i] = reason
                req.finish_reason = reason
                self.scheduler.finish(req)
        nxt = self._make_plan()
        if nxt.scheduled:
            # queued behind the running step at once: ids still unknown come from that step's output on the device
            self._inflight = self._launch(nxt, {id(s.request): i for i, s in enumerate(sampling)})
        elif nxt.early_results:
            self._next = nxt
        ids = self._read_sampled(sampled)                 # waits for the step
        stops = []
        for i, (s, tok) in enumerate(zip(sampling, ids)):
            if filed[i] is None:
                continue
            req = s.request
            req.token_ids[filed[i]] = tok
            if _is_stop_token(req.params, tok):
                stops.append(i)
                req.finish_reason = FinishReason.STOP    # the stop token wins over a length limit, as in the reference
                if i not in ended:
                    # whatever its state (it may have lost its pages in this very round); if the queued step
                    # computes one more token for it, that is dropped there
                    self.scheduler.finish(req)
        for i, (s, tok) in enumerate(zip(sampling, ids)):
            if filed[i] is None:
                continue
            req = s.request
            stop = i in stops
            results.append(EngineStepResult(req.request_id, tok, stop or i in ended,
                                            FinishReason.STOP if stop else ended.get(i), req.num_prompt_tokens,
                                            req.num_generated_tokens))
        return results

    def _launch(self, plan: "_Plan", sampled_before: Optional[Dict[int, int]] = None):
        """Queue a prepared step and its sampling on the device; returns (plan, handle of the sampled
        token ids for :meth:`_read_sampled`, or None if no request of the step samples).
        ``sampled_before``: id(request) -> row of the running step's sampler output, for the
        requests whose newest token is still being sampled."""
        self._fill_unknown_tokens(plan, sampled_before)
        sampling = plan.sampling
        sampler_inputs = None
        if sampling:                                      # uploaded ahead of the model's kernels
            if plan.sampler_staged is None:
                self._stage_plan(plan)
            sampler_inputs = self.sampler.send(plan.sampler_staged)
            plan.sampler_staged = None
        logits = self.runner.launch(plan.prepared)
        if not sampling:
            return plan, None
        if self.on_logits is not None:
            self.on_logits(sampling, logits)
        n = len(sampling)
        if n > self._sampled_dev.numel():
            raise RuntimeError(f"{n} requests sample in one step, more than max_bs={self.config.max_bs}")
        sampled = self.sampler.launch(logits, sampler_inputs, out=self._sampled_dev)
        host = self._sampled_host[self._sampled_turn]
        self._sampled_turn ^= 1
        host[:n].copy_(sampled, non_blocking=True)        # in stream order: before the next step's sampling overwrites it
        if host.is_pinned():
            done = torch.cuda.Event()
            done.record()
        else:
            done = None
        return plan, (host, n, done)

    @staticmethod
    def _read_sampled(handle) -> List[int]:
        host, n, done = handle
        if done is not None:
            done.synchronize()
        return host[:n].tolist()

    def _step_in_turn(self) -> List[EngineStepResult]:
        """Schedule, run, wait, file the tokens: one thing after the other."""
        plan = self._make_plan()
        results = plan.early_results
        if not plan.scheduled:
            return results
        _, sampled = self._launch(plan)
        if sampled is None:
            return results
        for s, tok in zip(plan.sampling, self._read_sampled(sampled)):
            req = s.request
            self.scheduler.append_token(req, tok)
            done, reason = self._is_finished(req)
            if done:
                req.finish_reason = reason
                self.scheduler.finish(req)
            results.append(EngineStepResult(req.request_id, tok, done, reason, req.num_prompt_tokens,
                                            req.num_generated_tokens))
        return results

    def _make_plan(self) -> "_Plan":
        """Schedule a step and do its host work.  Tokens that are still being sampled are packed as
        unknown and filled in by :meth:`_fill_unknown_tokens`."""
        scheduled = self.scheduler.schedule()
        early = [EngineStepResult(req.request_id, -1, True, req.finish_reason, req.num_prompt_tokens,
                                  req.num_generated_tokens) for req in self.scheduler.finished_by_scheduler]
        self.scheduler.finished_by_scheduler.clear()
        plan = _Plan(scheduled, early)
        self._pack_plan(plan)
        return plan

    def _pack_plan(self, plan: "_Plan") -> None:
        scheduled = plan.scheduled
        plan.sampling = [s for s in scheduled if s.samples]
        plan.sample_positions = [s.request.num_tokens for s in plan.sampling]
        plan.prepared = None
        plan.sampler_staged = None
        if scheduled:
            entries = [StepEntry(s.request.cache, s.request.token_ids[s.start:s.start + s.num_tokens],
                                 [s.num_tokens - 1] if s.samples else []) for s in scheduled]
            plan.prepared = self.runner.prepare(entries, allow_unknown=True)
            self._stage_plan(plan)

    def _stage_plan(self, plan: "_Plan") -> None:
        """Put the step's batch description and its sampling parameters into pinned memory, so that
        its launch only has to fill in late token ids and queue two copies."""
        self.runner.stage(plan.prepared)
        if plan.sampling:
            plan.sampler_staged = self.sampler.stage([s.request.params for s in plan.sampling],
                                                     [s.request.seed for s in plan.sampling], plan.sample_positions)

    def _fill_unknown_tokens(self, plan: "_Plan", sampled_before: Optional[Dict[int, int]] = None) -> None:
        """Ids the host has learnt since the step was packed are written in; one that is still being
        sampled (the newest token of a request of the running step) is left to the device."""
        for k, (b, j) in enumerate(plan.prepared.unknown_tokens()):
            s = plan.scheduled[b]
            req = s.request
            token = req.token_ids[s.start + j]
            if token != UNKNOWN_TOKEN:
                plan.prepared.fill_token(k, token)
                continue
            row = None if sampled_before is None else sampled_before.get(id(req))
            if row is None or s.start + j != req.num_tokens - 1:
                raise RuntimeError(f"request {req.request_id!r}: a token of the step is still unknown")
            plan.prepared.feed_token(k, row)
        plan.prepared.all_tokens_known()

    def _drop_from_next(self, req: Request) -> None:
        """A request of the prepared step has ended after all: pack the step again without it."""
        plan = self._next
        if plan is not None and any(s.request is req for s in plan.scheduled):
            plan.scheduled = [s for s in plan.scheduled if s.request is not req]
            self._pack_plan(plan)

    def _ends_by_length(self, req: Request) -> Optional[FinishReason]:
        """The length rules of :meth:`_is_finished`; they need no token ids, only counts."""
        p = req.params
        if ((p.max_tokens and req.num_tokens >= p.max_tokens)
                or (p.max_new_tokens and req.num_generated_tokens >= p.max_new_tokens)
                or req.num_tokens >= self.config.context_len):
            return FinishReason.LENGTH
        return None

    def _is_finished(self, req: Request):
        """The reference's rules in its order (ullm/core/engine.py:175-200)."""
        p = req.params
        if _is_stop_token(p, req.token_ids[-1]):
            return True, FinishReason.STOP
        if p.max_tokens and req.num_tokens >= p.max_tokens:
            return True, FinishReason.LENGTH
        if p.max_new_tokens and req.num_generated_tokens >= p.max_new_tokens:
            return True, FinishReason.LENGTH
        if req.num_tokens >= self.config.context_len:
            return True, FinishReason.LENGTH
        return False, None


def _is_stop_token(params: SamplingParams, token: int) -> bool:
    """The request's eos_token_id or one of its stop_token_ids, unless it ignores them."""
    if params.ignore_eos:
        return False
    return token == params.eos_token_id or token in params.stop_token_ids
