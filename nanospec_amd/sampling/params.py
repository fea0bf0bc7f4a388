"""Sampling options of a request, with the reference's names, meanings and defaults
(sched/scheduler.py:17-42; the fields that only speculative decoding reads are left out)."""

from __future__ import annotations

from dataclasses import dataclass


@dataclass(frozen=True)
class SamplingParams:
    max_tokens: int = 128  # stop after this many output tokens
    temperature: float = 0.0  # 0 = greedy: arg-max of the raw 32-bit logits
    top_k: int = 0  # keep the k most likely tokens (after the temperature); 0 = off
    top_p: float = 1.0  # keep tokens while the probability mass ranked before them is <= top_p; 1 = off
    seed: int | None = None  # seed of the request's own random numbers; None = not reproducible
    logprobs: bool = False  # fill Request.logprobs

    def __post_init__(self) -> None:
        if self.max_tokens < 1:
            raise ValueError(f"max_tokens must be at least 1, got {self.max_tokens}")
        if self.temperature < 0:
            raise ValueError(f"temperature must not be negative, got {self.temperature}")
        if self.top_k < 0 or not 0.0 < self.top_p <= 1.0:
            raise ValueError(f"top_k must be >= 0 and top_p in (0, 1], got {self.top_k}, {self.top_p}")


@dataclass(slots=True)
class TokenInfo:
    """Per emitted token (reference: sched/scheduler.py:45-52 without the speculative fields)."""

    token: int
    logprob: float  # log p(token) under the raw logits: temperature 1, no top-k / top-p
    sample_logprob: float  # log-probability under the distribution it was drawn from; 0 when greedy
