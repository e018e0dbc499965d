"""Per-request sampling options.

Reference: minivllm/config/sampling.py:4-10 — the same five names and defaults. ``seed``
is an addition: the reference draws unseeded.

Meaning of the options here:
  temperature  0 picks the arg-max (ties go to the lowest id). A positive value divides the
               logits by it (minivllm/models/layers/sampler.py:15-16) and one token is drawn
               from the softmax of the result. The reference falls through to ``argmax``
               whenever neither top_k nor top_p is set (sampler.py:31); here a positive
               temperature always draws.
  top_k        0 keeps all tokens, k > 0 keeps the k largest logits (sampler.py:18-27).
  top_p        1.0 keeps all, p < 1 keeps the smallest set of most likely tokens whose
               probabilities sum to at least p.
  max_tokens   the most tokens generated (minivllm/scheduler/scheduler.py:105).
  ignore_eos   go on past an end-of-sequence token (scheduler.py:106).
  seed         seed of the request's own random stream; None takes the engine's seed and
               the request's id.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Optional


@dataclass
class SamplingParams:
    temperature: float = 1.0
    max_tokens: int = 512
    ignore_eos: bool = False
    top_k: int = 0
    top_p: float = 1.0
    seed: Optional[int] = None

    def __post_init__(self) -> None:
        self.validate()

    def validate(self) -> None:
        if not (self.temperature >= 0.0):
            raise ValueError(f"temperature must be >= 0, got {self.temperature}")
        if self.max_tokens < 1:
            raise ValueError(f"max_tokens must be >= 1, got {self.max_tokens}")
        if self.top_k < 0:
            raise ValueError(f"top_k must be >= 0, got {self.top_k}")
        if not (0.0 < self.top_p <= 1.0):
            raise ValueError(f"top_p must be in (0, 1], got {self.top_p}")

    @property
    def greedy(self) -> bool:
        return self.temperature == 0.0
