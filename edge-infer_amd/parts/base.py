"""Interfaces of the parts and the context a step hands to them.

Every part is built as `cls(spec, hidden_size, params, dtype, device, **deps)`
from its own spec (all sizes and constants are fields of the spec) and the tensors
named by `cls.parameters(spec, hidden_size)`.  No part knows which model it is in.

mixer         parameters(), cache_request(spec) -> KVRequest | StateRequest | None,
              forward(ctx, x[N, H], entry) -> delta [N, H] or [splits, N, H]
feed_forward  parameters(), forward(ctx, x[N, H]) -> delta
norm          parameters(), add_norm(ctx, residual, delta, out_name, rows=None)
position      table(device) -> whatever its mixers read (a float32 angle table)
block         parameters(), forward(ctx, residual, pending, entry) -> pending

`residual` is the float32 stream [N, H]; `pending` is a delta not yet added to it
(the next norm adds it while it reads the row, which saves one pass over memory).
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Dict, Optional, Tuple

import torch


@dataclass(frozen=True)
class KVRequest:
    """Keys and values for every position (or the last `window`) of a sequence."""
    n_kv_heads: int
    head_dim: int
    window: Optional[int] = None


@dataclass(frozen=True)
class StateRequest:
    """A float32 tensor of fixed shape per sequence, zero when the sequence starts."""
    shape: Tuple[int, ...]


class Workspace:
    """Named device buffers that live across steps and only ever grow."""

    def __init__(self, device):
        self.device = device
        self._buffers: Dict[str, torch.Tensor] = {}

    def get(self, name: str, shape, dtype) -> torch.Tensor:
        count = 1
        for extent in shape:
            count *= int(extent)
        held = self._buffers.get(name)
        if held is None or held.dtype != dtype or held.numel() < count:
            held = torch.empty(max(count, 1), dtype=dtype, device=self.device)
            self._buffers[name] = held
        return held[:count].view(*shape)

    def bytes(self) -> int:
        return sum(b.numel() * b.element_size() for b in self._buffers.values())


class StepContext:
    """What one step gives to the parts: row metadata on the device, the cache
    entries, the workspace and the kind of step."""

    def __init__(self, *, dtype, device, n_rows, n_seqs, decode, meta, cache, workspace,
                 max_context):
        self.dtype = dtype            # storage type of activations and cache
        self.device = device
        self.n_rows = n_rows          # packed rows of this step (padding rows included)
        self.n_seqs = n_seqs
        self.decode = decode          # every sequence advances by exactly one token
        self.meta = meta              # engine.batch.DeviceMeta
        self.cache = cache            # cache.storage.SessionCache
        self.workspace = workspace
        self.max_context = max_context  # longest sequence after this step (host value)

    def buffer(self, name, shape, dtype=None):
        return self.workspace.get(name, shape, self.dtype if dtype is None else dtype)
