"""Device storage of the cache and its bookkeeping for one session.

The model's schedule names cache entries; the mixer that writes an entry says what
it needs (`KVRequest`: keys and values per position, perhaps only a window of them;
`StateRequest`: a tensor of fixed size per sequence).  Entries with the same needs
form a group with storage of its own:

  key/value group   k: [entries, pages, kv_heads, 64, head_dim], v: the same with the
                    group's value width, in the storage type; a page pool, and per
                    slot the list of its pages
  state group       [entries, slots + 1, *shape] float32, zeroed when a slot is taken; the
                    last row is a spare that no sequence owns (padding of a fixed-size
                    batch points there, so kernels need no branch for it)

A slot is one live sequence.  Its length is the number of tokens it holds, which is
also the position of its next token.  Taking a slot leaves old bytes in place: only
lengths and page lists say what is valid (the reference's `clear()` likewise only
sets the length, runtime/src/inference.cpp:115-126).
"""
from __future__ import annotations

from typing import Dict, List, Sequence, Tuple

import numpy as np
import torch

from ..parts.base import KVRequest, StateRequest
from ..parts.registry import lookup
from .allocator import PAGE_TOKENS, CacheFull, PagePool, SequencePages, SlotTable, pages_for


class CacheLayout:
    """Which cache entries exist and how they group, derived from a model spec."""

    def __init__(self, spec):
        self.kv_groups: List[Tuple[KVRequest, List[int]]] = []
        self.state_groups: List[Tuple[StateRequest, List[int]]] = []
        self.entry_group: Dict[int, Tuple[str, int, int]] = {}  # cache id -> (kind, group, index)
        for entry in spec.schedule:
            if not entry.writes_cache:
                continue
            layer = spec.layers[entry.layer]
            block_cls = lookup("block", layer.block)
            mixer_spec = block_cls.mixer_spec(layer)
            request = lookup("mixer", mixer_spec.kind).cache_request(mixer_spec)
            if request is None:
                continue
            groups = self.kv_groups if isinstance(request, KVRequest) else self.state_groups
            kind = "kv" if isinstance(request, KVRequest) else "state"
            for index, (held, entries) in enumerate(groups):
                if held == request:
                    self.entry_group[entry.cache] = (kind, index, len(entries))
                    entries.append(entry.cache)
                    break
            else:
                self.entry_group[entry.cache] = (kind, len(groups), 0)
                groups.append((request, [entry.cache]))


class SessionCache:
    def __init__(self, layout: CacheLayout, max_tokens: int, n_slots: int, dtype, device,
                 max_positions: int):
        self.layout = layout
        self.dtype = dtype
        self.device = device
        self.n_pages = max(1, pages_for(max_tokens))
        self.n_slots = int(n_slots)
        self.slots = SlotTable(self.n_slots)
        self.lengths = [0] * self.n_slots
        self.max_seq_tokens = min(max_positions, self.n_pages * PAGE_TOKENS)
        self.table_width = pages_for(self.max_seq_tokens)
        self.kv_pools: List[PagePool] = []
        self.kv_pages: List[SequencePages] = []
        self.kv_k: List[torch.Tensor] = []
        self.kv_v: List[torch.Tensor] = []
        for request, entries in layout.kv_groups:
            pool = PagePool(self.n_pages)
            self.kv_pools.append(pool)
            self.kv_pages.append(SequencePages(pool, self.n_slots, window=request.window))
            shape = (len(entries), self.n_pages, request.n_kv_heads, PAGE_TOKENS)
            value_dim = request.head_dim if request.value_dim is None else request.value_dim
            self.kv_k.append(torch.empty(shape + (request.head_dim,), dtype=dtype, device=device))
            self.kv_v.append(torch.empty(shape + (value_dim,), dtype=dtype, device=device))
        self._page_mirror: List[Dict[int, tuple]] = [{} for _ in self.kv_pages]
        self.states: List[torch.Tensor] = []
        self._state_copies: List[torch.Tensor] = []     # [slots, entries, *shape], see save_states
        for request, entries in layout.state_groups:
            self.states.append(torch.zeros((len(entries), self.n_slots + 1) + tuple(request.shape),
                                           dtype=torch.float32, device=device))
            self._state_copies.append(torch.empty((self.n_slots, len(entries))
                                                  + tuple(request.shape),
                                                  dtype=torch.float32, device=device))

    # -- slots -------------------------------------------------------------
    def acquire(self) -> int:
        slot = self.slots.acquire()
        self.lengths[slot] = 0
        for pages in self.kv_pages:
            pages.open(slot)
        for state in self.states:
            state[:, slot].zero_()
        return slot

    def release(self, slot: int) -> None:
        self.slots.release(slot)   # raises on a slot that is not live
        for pages in self.kv_pages:
            pages.close(slot)
        self.lengths[slot] = 0

    def release_all(self) -> None:
        for slot in self.slots.live_slots():
            self.release(slot)

    # -- growth ------------------------------------------------------------
    def check_growth(self, growth: Sequence[Tuple[int, int]]) -> None:
        """Raise, changing nothing, unless every (slot, new length) fits."""
        for slot, new_length in growth:
            if not self.slots.is_live(slot):
                raise ValueError(f"slot {slot} is not live")
            if new_length > self.max_seq_tokens:
                raise CacheFull(f"a sequence of {new_length} tokens exceeds the limit of "
                                f"{self.max_seq_tokens}")
        for pages in self.kv_pages:
            need = sum(pages.pages_needed(slot, new_length) for slot, new_length in growth)
            if need > pages.pool.n_free:
                raise CacheFull(f"{need} cache pages wanted, {pages.pool.n_free} free "
                                f"of {pages.pool.n_pages}")

    def grow(self, growth: Sequence[Tuple[int, int]]) -> None:
        self.check_growth(growth)
        for pages in self.kv_pages:
            for slot, new_length in growth:
                pages.grow(slot, new_length)

    def commit(self, growth: Sequence[Tuple[int, int]]) -> None:
        """The step has run: lengths advance, windows let go of dead pages."""
        for slot, new_length in growth:
            self.lengths[slot] = new_length
            for pages in self.kv_pages:
                pages.trim(slot, new_length)

    # -- fixed-size state: what a step may change in place ------------------
    def save_states(self, slots: torch.Tensor) -> None:
        """Copy the state rows of these slots (int32 on the device, one per live sequence of
        the step about to run) aside.  Mixers update state in place while a step runs; keys
        and values of a failed step lie beyond the committed lengths and are simply written
        again, but state has no such place, so a failed step puts these copies back."""
        for state, copy in zip(self.states, self._state_copies):
            torch.index_select(state.transpose(0, 1), 0, slots, out=copy[:slots.numel()])

    def restore_states(self, slots: torch.Tensor) -> None:
        """Put back what `save_states` copied for the same slots."""
        for state, copy in zip(self.states, self._state_copies):
            state.transpose(0, 1).index_copy_(0, slots.long(), copy[:slots.numel()])

    # -- views -------------------------------------------------------------
    def kv(self, cache_id: int):
        kind, group, index = self.layout.entry_group[cache_id]
        if kind != "kv":
            raise KeyError(f"cache entry {cache_id} holds no keys and values")
        return group, self.kv_k[group][index], self.kv_v[group][index]

    def state(self, cache_id: int) -> torch.Tensor:
        """[slots + 1, *shape] float32 of a fixed-size state entry (row = slot; the last row
        is the spare one)."""
        kind, group, index = self.layout.entry_group[cache_id]
        if kind != "state":
            raise KeyError(f"cache entry {cache_id} holds no fixed-size state")
        return self.states[group][index]

    def page_rows(self, group: int, slots: Sequence[int], n_rows: int) -> np.ndarray:
        """int32 [n_rows, table_width]: logical page -> physical page (-1: none) for
        the given slots; rows beyond them are padding."""
        table = np.full((n_rows, self.table_width), -1, dtype=np.int32)
        pages, mirror = self.kv_pages[group], self._page_mirror[group]
        for i, slot in enumerate(slots):
            row = pages.row(slot)
            # a slot's row is kept as an array and refreshed only when its pages change (they
            # change when the sequence passes a page boundary, not with every token)
            version = pages.version(slot)
            kept = mirror.get(slot)
            if kept is None or kept[0] != version:
                kept = mirror[slot] = (version, np.asarray(row, dtype=np.int32))
            table[i, :kept[1].size] = kept[1]
        return table

    def bytes(self) -> int:
        total = 0
        for tensor in self.kv_k + self.kv_v + self.states + self._state_copies:
            total += tensor.numel() * tensor.element_size()
        return total

    def check(self) -> None:
        self.slots.check()
        for pool, pages in zip(self.kv_pools, self.kv_pages):
            pool.check()
            if pages.held() != pool.n_pages - pool.n_free:
                raise AssertionError("pages held by sequences and pages missing from the pool differ")
