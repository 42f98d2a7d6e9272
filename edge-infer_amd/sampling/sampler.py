"""Draws tokens from float32 logits on the GPU (see csrc/sampling.hip).

A request's draws depend only on (seed, its stream number, its step counter), so it
samples the same tokens alone or in any batch.
"""
from __future__ import annotations

from typing import List, Sequence

import torch

from ..csrc import lib
from .params import SamplingParams


class Sampler:
    def __init__(self, device):
        self.device = torch.device(device)
        self._tokens = torch.empty(1024, dtype=torch.int32, device=self.device)
        self._probabilities = torch.empty(1024, dtype=torch.float32, device=self.device)
        self._meta = torch.empty(2048, dtype=torch.int32, device=self.device)
        # stream numbers and counters travel through pinned memory; two buffers in turn, so
        # that filling one does not disturb a copy of the other that is still queued
        self._meta_host = [torch.empty(2048, dtype=torch.int32, pin_memory=True) for _ in range(2)]
        self._meta_turn = 0
        self._partial = None          # scratch of the greedy search over a wide vocabulary
        self._scratch = None          # zeroed scratch of sampling from a wide vocabulary
        self._last_rows = 0

    def _reserve(self, rows: int) -> None:
        if self._tokens.numel() < rows:
            self._tokens = torch.empty(rows, dtype=torch.int32, device=self.device)
            self._probabilities = torch.empty(rows, dtype=torch.float32, device=self.device)
            self._meta = torch.empty(2 * rows, dtype=torch.int32, device=self.device)
            self._meta_host = [torch.empty(2 * rows, dtype=torch.int32, pin_memory=True)
                               for _ in range(2)]

    def sample_device(self, logits: torch.Tensor, params: SamplingParams, streams: Sequence[int],
                      counters: Sequence[int]) -> torch.Tensor:
        """int32 tokens [rows] on the device (a view that the next call overwrites)."""
        rows, vocab = logits.shape
        params.validate(vocab)
        self._reserve(rows)
        tokens = self._tokens[:rows]
        probabilities = self._probabilities[:rows]
        if params.is_greedy(vocab):
            need = lib.argmax_partial_size(rows, vocab)
            if need and (self._partial is None or self._partial.numel() < need):
                self._partial = torch.empty(need, dtype=torch.float32, device=self.device)
            lib.argmax(logits, tokens, probabilities, self._partial if need else None)
        else:
            if len(streams) != rows or len(counters) != rows:
                raise ValueError("one stream number and one counter per row are needed")
            host = self._meta_host[self._meta_turn]
            self._meta_turn ^= 1
            host[:2 * rows] = torch.tensor(list(streams) + list(counters), dtype=torch.int32)
            self._meta[:2 * rows].copy_(host[:2 * rows], non_blocking=True)
            need = lib.sample_scratch_size(rows, vocab)
            if need and (self._scratch is None or self._scratch.numel() < need):
                self._scratch = torch.zeros(need, dtype=torch.int32, device=self.device)
            lib.sample(logits, params.temperature, params.top_p, params.top_k, params.seed,
                       self._meta[:rows], self._meta[rows:2 * rows], tokens, probabilities,
                       self._scratch if need else None)
        return tokens

    def __call__(self, logits, params, streams, counters) -> List[int]:
        """Tokens as Python ints (one device-to-host copy, which also waits for the step)."""
        tokens = self.sample_device(logits, params, streams, counters)
        self._last_rows = logits.shape[0]
        return tokens.tolist()

    def probabilities(self) -> List[float]:
        """Probability of each token of the last call within its filtered distribution."""
        return self._probabilities[:self._last_rows].tolist()
