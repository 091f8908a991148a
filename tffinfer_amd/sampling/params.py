"""Sampling options, with the names and meanings of the reference's
SamplingConfig (src/core/sampler/LLMSampler.h:55-63): ``_type``,
``_temperature``, ``_top_k``, ``_top_p``, ``_min_p``, ``_repetition_penalty``,
``_seed`` there, the same without the underscore here."""
from __future__ import annotations

from dataclasses import dataclass

#: strategy names of the reference (src/core/sampler/LLMSampler.h:18-24)
STRATEGIES = ("default", "unknown", "greedy", "random", "top_k", "top_p")


@dataclass
class SamplingConfig:
    """``type`` 'greedy' (and 'default', as the reference's ``sample()`` always
    takes the argmax, src/core/sampler/LLMSampler.cpp:13-19) picks the first
    maximum.  'random', 'top_k' and 'top_p' draw from softmax(logits /
    temperature), restricted to the ``top_k`` most likely tokens (0: off), to
    the most likely tokens whose mass reaches ``top_p`` (1: off) and to tokens
    with probability at least ``min_p`` times the largest (0: off).
    ``temperature`` 0 also means greedy.  ``repetition_penalty`` divides the
    positive and multiplies the other logits of tokens already in the prompt or
    the output (LLMSampler.cpp:21-34).  The draw for output token i of a
    request depends only on (seed, i), not on what else is in the batch.
    """
    type: str = "greedy"
    temperature: float = 1.0
    top_k: int = 0
    top_p: float = 1.0
    min_p: float = 0.0
    repetition_penalty: float = 1.0
    seed: int = 0

    def __post_init__(self):
        if self.type not in STRATEGIES or self.type == "unknown":
            raise ValueError(f"unknown sampling strategy '{self.type}'; known: {STRATEGIES}")
        if self.temperature < 0:
            raise ValueError("temperature must not be negative")
        if self.top_k < 0 or not (0 < self.top_p <= 1) or not (0 <= self.min_p <= 1):
            raise ValueError("top_k >= 0, 0 < top_p <= 1 and 0 <= min_p <= 1 are required")
        if self.repetition_penalty <= 0:
            raise ValueError("repetition_penalty must be positive")

    @property
    def greedy(self) -> bool:
        return self.type in ("greedy", "default") or self.temperature == 0

    def effective(self):
        """(temperature, top_k, top_p, min_p) the kernel gets; temperature 0 = argmax."""
        if self.greedy:
            return 0.0, 0, 1.0, 0.0
        return float(self.temperature), int(self.top_k), float(self.top_p), float(self.min_p)
