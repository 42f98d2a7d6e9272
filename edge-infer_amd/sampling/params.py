"""Sampling options and their validation.

Rules of the reference (operators/src/cuda/execution.cu:455-462): top_k >= 1,
temperature and top_p finite, 0 < top_p <= 1, min(top_k, vocab) <= 1024.
`temperature <= 0` or `min(top_k, vocab) == 1` means greedy (argmax, ties to the
lowest index).  The defaults are those of the reference's Python
`Session.generate` (bindings/python/model_bridge.cpp:248-252).
"""
from __future__ import annotations

import math
from dataclasses import dataclass

MAX_TOP_K = 1024


@dataclass(frozen=True)
class SamplingParams:
    temperature: float = 1.0
    top_p: float = 0.9
    top_k: int = 1
    seed: int = 0

    def validate(self, vocab_size: int) -> None:
        if vocab_size < 1:
            raise ValueError("sampling needs a vocabulary")
        if isinstance(self.top_k, bool) or not isinstance(self.top_k, int) or self.top_k < 1:
            raise ValueError(f"top_k must be a positive integer, got {self.top_k!r}")
        if not math.isfinite(self.temperature):
            raise ValueError("temperature must be finite")
        if not math.isfinite(self.top_p) or not 0.0 < self.top_p <= 1.0:
            raise ValueError(f"top_p must lie in (0, 1], got {self.top_p!r}")
        if min(self.top_k, vocab_size) > MAX_TOP_K:
            raise ValueError(f"min(top_k, vocabulary) must not exceed {MAX_TOP_K}")

    def is_greedy(self, vocab_size: int) -> bool:
        return self.temperature <= 0.0 or min(self.top_k, vocab_size) == 1
