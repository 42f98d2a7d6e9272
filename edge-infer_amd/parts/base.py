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
    """Keys and values for every position (or the last `window`) of a sequence: pages
    [kv_heads, 64, head_dim] of keys and [kv_heads, 64, value_dim] of values (`value_dim`
    None: as wide as the keys)."""
    n_kv_heads: int
    head_dim: int
    window: Optional[int] = None
    value_dim: Optional[int] = None


@dataclass(frozen=True)
class StateRequest:
    """A float32 tensor of fixed shape per sequence, zero when the sequence starts."""
    shape: Tuple[int, ...]


class Workspace:
    """Named device buffers of a step.

    Without `start` (a part run on its own): one buffer per name that lives across steps
    and only ever grows.  Between `start(signature)` and `finish()`: the first step of a
    signature runs on such buffers and records when each value is asked for and when it
    is `release`d; from that the planner lays the values out in one arena so that values
    whose lifetimes do not overlap share storage (the reference plans its decoder
    buffers the same way, runtime/include/execution/decoder.hpp:46-58 over
    core/include/execution/workspace_plan.hpp); later steps of that signature take their
    buffers from the arena.  A step that asks for something else than was recorded (a
    name, an order, a larger size) is served from named buffers from there on and its
    signature is planned anew next time.  A name that is asked for again while still live
    stands for the same storage until then, so the earlier value ends there.

    `start(signature, scale)`: a signature may stand for a class of steps (prompt steps of
    about so many rows); the recorded sizes are then multiplied by `scale`, the ratio of the
    class's largest step to the recorded one, so that every step of the class finds room at
    the planned places.  At most `MAX_PLANS` plans are kept; the one unused for longest goes
    first.  `bind(name, tensor)`: requests for that name are served from the caller's tensor
    and are not part of any plan (several workspaces can share one large buffer this way)."""

    MAX_PLANS = 32

    def __init__(self, device):
        self.device = device
        self._buffers: Dict[str, torch.Tensor] = {}
        self._arena: Optional[torch.Tensor] = None
        self._plans: Dict[object, "_StepLayout"] = {}
        self._signature = None
        self._layout: Optional["_StepLayout"] = None     # replaying this layout
        self._events: Optional[list] = None               # recording these events
        self._cursor = 0
        self._names: Dict[int, str] = {}                  # data pointer -> name, this step
        self._scale = 1.0
        self._bound: Dict[str, torch.Tensor] = {}

    def bind(self, name: str, tensor: Optional[torch.Tensor]) -> None:
        """Serve requests for `name` from `tensor` (None: no longer)."""
        if tensor is None:
            self._bound.pop(name, None)
        else:
            self._bound[name] = tensor

    def clear(self) -> None:
        """Forget every plan and give all storage back."""
        self._buffers.clear()
        self._plans.clear()
        self._arena = None
        self._signature = self._layout = self._events = None

    # -- one step ------------------------------------------------------------
    def start(self, signature, scale: float = 1.0) -> None:
        self._signature = signature
        self._layout = self._plans.pop(signature, None)
        if self._layout is not None:
            self._plans[signature] = self._layout         # most recently used: last
        self._events = [] if self._layout is None else None
        self._cursor = 0
        self._scale = max(1.0, float(scale))
        self._names.clear()

    def finish(self) -> None:
        if self._events is not None:
            layout = _StepLayout.from_recording(self._events, self._scale)
            while len(self._plans) >= self.MAX_PLANS:
                self._plans.pop(next(iter(self._plans)))
            self._plans[self._signature] = layout
            if self._arena is None or self._arena.numel() < layout.arena.arena_bytes:
                self._arena = torch.empty(max(layout.arena.arena_bytes, 256), dtype=torch.uint8,
                                          device=self.device)
                for other in self._plans.values():
                    other.views.clear()               # they pointed into the old arena
            self._buffers.clear()    # what the step handed out stays alive with its holders
        self._signature = self._layout = self._events = None

    def abort(self) -> None:
        """The step failed: nothing of it is kept."""
        self._signature = self._layout = self._events = None

    def _diverged(self) -> None:
        """The step does not follow its recording: named buffers from here on."""
        self._plans.pop(self._signature, None)
        self._layout = None

    # -- buffers ---------------------------------------------------------------
    def get(self, name: str, shape, dtype) -> torch.Tensor:
        count = 1
        for extent in shape:
            count *= int(extent)
        bound = self._bound.get(name)
        if bound is not None:
            if bound.dtype != dtype or bound.numel() < count:
                raise ValueError(f"the buffer bound to '{name}' holds {bound.numel()} elements of "
                                 f"{bound.dtype}; {count} of {dtype} are wanted")
            return bound.view(-1)[:count].view(*shape)
        layout = self._layout
        if layout is not None:
            index = self._cursor
            if index < len(layout.events) and layout.events[index][0] == name:
                _, nbytes, key = layout.events[index]
                if nbytes is not None and count * dtype.itemsize <= nbytes:
                    self._cursor = index + 1
                    view = layout.views.get(index)
                    if view is None or view.dtype != dtype or tuple(view.shape) != tuple(shape):
                        offset = layout.arena.offset(key)
                        raw = self._arena[offset:offset + count * dtype.itemsize]
                        view = raw.view(dtype).view(*shape)
                        layout.views[index] = view
                    self._names[view.data_ptr()] = name
                    return view
            self._diverged()
        if self._events is not None:
            self._events.append((name, max(count, 1) * dtype.itemsize))
        held = self._buffers.get(name)
        if held is None or held.dtype != dtype or held.numel() < count:
            held = torch.empty(max(count, 1), dtype=dtype, device=self.device)
            self._buffers[name] = held
        if self._signature is not None:
            self._names[held.data_ptr()] = name
        return held[:count].view(*shape)

    def release(self, which) -> None:
        """The value last asked for under a name (given as the name, or as the tensor that
        `get` returned) is not read any more.  Anything else is ignored."""
        if self._signature is None or which is None:
            return
        name = which if isinstance(which, str) else self._names.get(which.data_ptr())
        if name is None:
            return
        layout = self._layout
        if layout is not None:
            index = self._cursor
            if index < len(layout.events) and layout.events[index] == (name, None, None):
                self._cursor = index + 1
            else:
                self._diverged()
        elif self._events is not None:
            self._events.append((name, None))

    def bytes(self) -> int:
        arena = 0 if self._arena is None else self._arena.numel()
        return arena + sum(b.numel() * b.element_size() for b in self._buffers.values())


class _StepLayout:
    """The recorded order of a step's requests and releases, and the plan made of it."""

    def __init__(self, events, arena):
        self.events = events      # (name, bytes, layout key) for a request, (name, None, None)
        self.arena = arena        # cache.workspace.ArenaLayout
        self.views: Dict[int, torch.Tensor] = {}

    @classmethod
    def from_recording(cls, recorded, scale: float = 1.0):
        """recorded: (name, bytes) for each request and (name, None) for each release, in
        order; a value lives from its request to the event before its release (or before
        the next request of its name), or to the end.  Sizes are multiplied by `scale`."""
        from ..cache.workspace import Lifetime, lay_out
        needs = []
        if scale > 1.0:
            recorded = [(name, None if nbytes is None else int(-(-nbytes * scale // 1)))
                        for name, nbytes in recorded]
        live: Dict[str, list] = {}        # name -> [layout key, bytes, tick of the request]
        events = []
        counts: Dict[str, int] = {}
        for tick, (name, nbytes) in enumerate(recorded):
            if name in live:              # released, or asked for again: the value ends
                key, size, first = live.pop(name)
                needs.append(Lifetime(key, size, first, max(first, tick - 1)))
            if nbytes is None:
                events.append((name, None, None))
                continue
            key = f"{name}#{counts.get(name, 0)}"
            counts[name] = counts.get(name, 0) + 1
            live[name] = [key, nbytes, tick]
            events.append((name, nbytes, key))
        for key, size, first in live.values():    # never released: live to the step's end
            needs.append(Lifetime(key, size, first, len(recorded)))
        return cls(events, lay_out(needs))


class StepContext:
    """What one step gives to the parts: row metadata on the device, the cache
    entries, the workspace and the kind of step."""

    def __init__(self, *, dtype, device, n_rows, n_seqs, decode, meta, cache, workspace,
                 max_context, context_bound=None, fixed_shape=False):
        self.dtype = dtype            # storage type of activations and cache
        self.device = device
        self.n_rows = n_rows          # packed rows of this step (padding rows included)
        self.n_seqs = n_seqs
        self.decode = decode          # every sequence advances by exactly one token
        self.meta = meta              # engine.batch.DeviceMeta
        self.cache = cache            # cache.storage.SessionCache
        self.workspace = workspace
        self.max_context = max_context  # longest sequence after this step (host value)
        # launch shapes must hold for sequences of up to this many tokens: the longest one of
        # the step, or more when the step is captured and replayed for longer contexts (then
        # `fixed_shape` is set, and what depends on the true lengths is read on the device)
        self.context_bound = max_context if context_bound is None else context_bound
        self.fixed_shape = fixed_shape
        self.sequences = ()             # engine.batch.SeqStep of every live sequence (host)
        self.notes = {}                 # what parts work out once a step and share between layers

    def buffer(self, name, shape, dtype=None):
        return self.workspace.get(name, shape, self.dtype if dtype is None else dtype)

    def release(self, *buffers) -> None:
        """These buffers (tensors that `buffer` returned, or their names) are not read any
        more in this step: their storage may serve a later request.  Optional: what is
        never released lives to the end of the step; None and tensors that are not the
        workspace's are ignored."""
        for which in buffers:
            self.workspace.release(which)
