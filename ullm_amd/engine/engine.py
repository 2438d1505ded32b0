"""The engine: scheduler + step function + sampler, one process, one GPU.

Reference: ullm/core/engine.py:24-238 (add_sequence, abort_sequence, step = schedule -> execute ->
update_from_output, finish rules) with ullm/core/model_runner.py:123-183,233-255 folded in (model
load, cache sizing from free memory).
"""
from __future__ import annotations

import logging
from typing import Dict, List, Optional, Sequence

import torch

from ..config.engine_config import EngineConfig
from ..sampling import Sampler, SamplingParams
from .loading import load_model
from .request import EngineStepResult, FinishReason, Request, RequestStatus, Scheduled
from .runner import ModelRunner, StepEntry
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


class Engine:
    def __init__(self, config: EngineConfig, model=None, env=None, model_config=None):
        """``model``/``env``/``model_config`` may be handed in already built (random weights on the
        device, tests); otherwise the folder ``config.model`` is loaded."""
        self.config = config
        logging.basicConfig(level=getattr(logging, config.log_level.upper(), logging.INFO))
        if model is None:
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
        self._arrivals = 0
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
        if params.eos_token_id == -1 and getattr(self.model_config, "eos_token_id", -1) is not None:
            params.eos_token_id = getattr(self.model_config, "eos_token_id", -1)
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

    def has_unfinished_requests(self) -> bool:
        return self.scheduler.has_unfinished()

    # ------------------------------------------------------------------ one step
    def step(self) -> List[EngineStepResult]:
        scheduled = self.scheduler.schedule()
        results: List[EngineStepResult] = []
        for req in self.scheduler.finished_by_scheduler:
            results.append(EngineStepResult(req.request_id, -1, True, req.finish_reason, req.num_prompt_tokens,
                                            req.num_generated_tokens))
        self.scheduler.finished_by_scheduler.clear()
        if not scheduled:
            return results
        entries = [StepEntry(s.request.cache, s.request.token_ids[s.start:s.start + s.num_tokens],
                             [s.num_tokens - 1] if s.samples else []) for s in scheduled]
        sampling = [s for s in scheduled if s.samples]
        prepared = None
        if sampling:                                      # uploaded ahead of the model step
            prepared = self.sampler.prepare([s.request.params for s in sampling], [s.request.seed for s in sampling],
                                            [s.request.num_tokens for s in sampling])
        logits = self.runner.step(entries)
        if sampling:
            if self.on_logits is not None:
                self.on_logits(sampling, logits)
            ids = self.sampler.sample(logits, prepared=prepared)
            for s, tok in zip(sampling, ids):
                req = s.request
                self.scheduler.append_token(req, tok)
                done, reason = self._is_finished(req)
                if done:
                    req.finish_reason = reason
                    self.scheduler.finish(req)
                results.append(EngineStepResult(req.request_id, int(tok), done, reason, req.num_prompt_tokens,
                                                req.num_generated_tokens))
        return results

    def _is_finished(self, req: Request):
        """The reference's rules in its order (ullm/core/engine.py:175-200)."""
        p = req.params
        if req.token_ids[-1] == p.eos_token_id and not p.ignore_eos:
            return True, FinishReason.STOP
        if p.max_tokens and req.num_tokens >= p.max_tokens:
            return True, FinishReason.LENGTH
        if p.max_new_tokens and req.num_generated_tokens >= p.max_new_tokens:
            return True, FinishReason.LENGTH
        if req.num_tokens >= self.config.context_len:
            return True, FinishReason.LENGTH
        return False, None
