"""Per-request sampling parameters, named and defaulted as the reference's
(ullm/core/common.py:7-19), plus a seed."""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import List, Optional


@dataclass
class SamplingParams:
    n: int = 1                              # carried, not used (the reference's engine ignores it too)
    temperature: float = 1.0                # 0 = greedy: first index of the largest logit
    top_p: float = 1.0
    top_k: int = -1                         # <= 0: the whole vocabulary
    min_p: float = 0.0

    max_tokens: Optional[int] = None        # cap on prompt + generated tokens (ullm/core/engine.py:184-189)
    max_new_tokens: Optional[int] = None    # cap on generated tokens
    stop: List[str] = field(default_factory=list)   # carried, not used (as in the reference)
    ignore_eos: bool = False
    eos_token_id: int = -1                  # -1: filled from the model's config when it names one
    stop_token_ids: List[int] = field(default_factory=list)   # further ids that end the request like eos_token_id

    seed: Optional[int] = None              # None: the engine's seed mixed with the request's order

    def __post_init__(self):
        if self.temperature < 0:
            raise ValueError("temperature must not be negative (0 selects greedy decoding)")
        if not (0.0 <= self.top_p <= 1.0):
            raise ValueError("top_p must lie in [0, 1]")
        if not (0.0 <= self.min_p <= 1.0):
            raise ValueError("min_p must lie in [0, 1]")
