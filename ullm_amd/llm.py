"""Python entry point in the reference's manner (ullm/llm.py:23-129): ``LLM(EngineConfig)``,
``generate`` for prompts given as token ids or text, ``abort``, ``shutdown``.

The reference's LLM is asynchronous because its engine lives in another process; here everything is
one process, so ``generate`` runs the engine until its requests are done and returns whole outputs,
and ``stream`` yields the reference's per-token ``GenerateOutput`` records as they are produced.
"""
from __future__ import annotations

import logging
import os
import uuid
from dataclasses import dataclass, field
from typing import Dict, Iterator, List, Optional, Sequence, Union

from .config.engine_config import EngineConfig
from .engine.engine import Engine
from .engine.request import EngineStepResult, FinishReason
from .sampling import SamplingParams

logger = logging.getLogger("ullm_amd")

Prompt = Union[str, Sequence[int]]


@dataclass
class GenerateOutput:
    """One generated token (reference: ullm/core/common.py:27-33), plus its id and request."""
    token_str: str
    is_finished: bool
    finish_reason: Optional[FinishReason]
    num_prompt_tokens: int
    num_generated_tokens: int
    token_id: int = -1
    sequence_id: str = ""


@dataclass
class RequestOutput:
    sequence_id: str
    prompt_token_ids: List[int]
    token_ids: List[int] = field(default_factory=list)
    text: Optional[str] = None
    finish_reason: Optional[FinishReason] = None

    @property
    def num_prompt_tokens(self) -> int:
        return len(self.prompt_token_ids)

    @property
    def num_generated_tokens(self) -> int:
        return len(self.token_ids)


def init_tokenizer(model: str):
    """Reference: ullm/llm.py:12-20.  Loaded only when text goes in or is asked for."""
    from transformers import AutoTokenizer
    tok = AutoTokenizer.from_pretrained(model, use_fast=False, trust_remote_code=False)
    if tok.pad_token is None:
        tok.pad_token = tok.eos_token
    if tok.unk_token is None:
        tok.unk_token = tok.eos_token
    return tok


class LLM:
    def __init__(self, config: EngineConfig, engine: Optional[Engine] = None):
        self.config = config
        self.engine = engine if engine is not None else Engine(config)
        self._tokenizer = None
        self._profiler = None

    # ------------------------------------------------------------------ text
    @property
    def tokenizer(self):
        if self._tokenizer is None:
            self._tokenizer = init_tokenizer(self.config.model)
        return self._tokenizer

    def tokenize(self, texts: List[str]) -> List[List[int]]:
        return self.tokenizer(texts)["input_ids"]

    def detokenize(self, token_ids: List[List[int]]) -> List[str]:
        return self.tokenizer.batch_decode(token_ids, skip_special_tokens=True)

    # ------------------------------------------------------------------ generation
    def _default_params(self) -> SamplingParams:
        return SamplingParams(**self.config.generation_defaults())

    def _submit(self, prompts, params, sequence_ids):
        single = isinstance(prompts, str) or (len(prompts) > 0 and isinstance(prompts[0], int))
        plist = [prompts] if single else list(prompts)
        if params is None:
            params = [self._default_params() for _ in plist]
        elif isinstance(params, SamplingParams):
            params = [SamplingParams(**vars(params)) for _ in plist]
        if len(params) != len(plist):
            raise ValueError("one SamplingParams per prompt is needed")
        if sequence_ids is None:
            sequence_ids = [uuid.uuid4().hex for _ in plist]
        elif isinstance(sequence_ids, str):
            sequence_ids = [sequence_ids]
        outs: Dict[str, RequestOutput] = {}
        uses_text = False
        for prompt, p, sid in zip(plist, params, sequence_ids):
            if isinstance(prompt, str):
                ids = self.tokenize([prompt])[0]
                uses_text = True
                if p.eos_token_id == -1 and self.tokenizer.eos_token_id is not None:
                    p.eos_token_id = self.tokenizer.eos_token_id      # reference: ullm/llm.py:93-94
            else:
                ids = list(prompt)
            req = self.engine.add_request(sid, ids, p)
            outs[sid] = RequestOutput(sid, list(req.token_ids[:req.num_prompt_tokens]))
        return outs, uses_text, single

    def stream(self, prompts: Union[Prompt, Sequence[Prompt]],
               params: Union[SamplingParams, Sequence[SamplingParams], None] = None,
               sequence_id: Union[str, Sequence[str], None] = None) -> Iterator[GenerateOutput]:
        """Yields one ``GenerateOutput`` per generated token of the submitted prompts."""
        outs, uses_text, _ = self._submit(prompts, params, sequence_id)
        pending = set(outs)
        while pending and self.engine.has_unfinished_requests():
            for r in self.engine.step():
                if r.seq_id not in pending:
                    continue
                text = self.detokenize([[r.new_token_id]])[0] if (uses_text and r.new_token_id >= 0) else ""
                if r.is_finished:
                    pending.discard(r.seq_id)
                yield GenerateOutput(text, r.is_finished, r.finish_reason,
                                     r.num_prompt_tokens if r.is_finished else 0,
                                     r.num_generated_tokens if r.is_finished else 0,
                                     r.new_token_id, r.seq_id)

    def generate(self, prompts: Union[Prompt, Sequence[Prompt]],
                 params: Union[SamplingParams, Sequence[SamplingParams], None] = None,
                 sequence_id: Union[str, Sequence[str], None] = None):
        """Runs the prompts to completion.  A single prompt returns one ``RequestOutput``; a list
        returns a list in the same order."""
        outs, uses_text, single = self._submit(prompts, params, sequence_id)
        pending = set(outs)
        while pending and self.engine.has_unfinished_requests():
            for r in self.engine.step():
                o = outs.get(r.seq_id)
                if o is None:
                    continue
                if r.new_token_id >= 0:
                    o.token_ids.append(r.new_token_id)
                if r.is_finished:
                    o.finish_reason = r.finish_reason
                    pending.discard(r.seq_id)
        result = list(outs.values())
        if uses_text:
            for o, text in zip(result, self.detokenize([o.token_ids for o in result])):
                o.text = text
        return result[0] if single else result

    def abort(self, sequence_id: str) -> None:
        self.engine.abort_request(sequence_id)

    def profile(self, action: str) -> None:
        """"start" / "stop" a torch profiler trace (host and device activity) into
        ``config.profile_dir``; needs ``config.profile`` (reference: ullm/core/worker.py:46-64,137-160)."""
        if not self.config.profile:
            raise RuntimeError("profiling is off: set EngineConfig.profile (--profile)")
        if action not in ("start", "stop"):
            raise ValueError('profile action must be "start" or "stop"')
        import torch
        if action == "start":
            if self._profiler is not None:
                logger.warning("profiler already started, ignoring")
                return
            os.makedirs(self.config.profile_dir, exist_ok=True)
            self._profiler = torch.profiler.profile(
                activities=[torch.profiler.ProfilerActivity.CPU, torch.profiler.ProfilerActivity.CUDA],
                on_trace_ready=torch.profiler.tensorboard_trace_handler(
                    os.path.abspath(self.config.profile_dir), worker_name=f"ullm_amd_{os.getpid()}", use_gzip=True),
                record_shapes=True)
            self._profiler.start()
        else:
            if self._profiler is None:
                logger.warning("profiler already stopped, ignoring")
                return
            self._profiler.stop()
            self._profiler = None

    def shutdown(self) -> None:
        """Nothing runs in the background; a step that was queued ahead for requests which have ended
        meanwhile is waited for, then the engine is let go (the reference's callers need no change)."""
        if self.engine is not None:
            self.engine.drain()
        self.engine = None
