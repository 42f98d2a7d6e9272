"""Offline planning of a step's workspace: values whose lifetimes do not overlap share
storage.

A request names a value, its size in bytes and the first and last step at which it is
used; the planner sorts requests by (first use, last use, name) and gives each the
smallest slot that is dead (its last value's last use lies strictly before the new
first use), large enough and aligned, or appends a new slot.  It allocates nothing: a
plan is a table of offsets into one arena.  Behaviour and checks follow the reference's
planner, core/include/execution/workspace_plan.hpp:138-252 (plan validation :32-60,
metrics :75-118).
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Dict, List, Optional


@dataclass(frozen=True)
class Allocation:
    name: str
    offset: int
    bytes: int
    first_use: int
    last_use: int
    alignment: int = 256


def _power_of_two(value: int) -> bool:
    return value > 0 and value & (value - 1) == 0


class WorkspacePlan:
    """Offsets of named values in an arena of `total_bytes`; construction checks that
    no two values that are live at the same time overlap in storage."""

    def __init__(self, allocations: List[Allocation], total_bytes: int):
        self.allocations = list(allocations)
        self.total_bytes = int(total_bytes)
        self._index: Dict[str, int] = {}
        for i, a in enumerate(self.allocations):
            if (not a.name or a.bytes <= 0 or a.first_use > a.last_use
                    or not _power_of_two(a.alignment) or a.offset % a.alignment
                    or a.offset < 0 or a.offset + a.bytes > self.total_bytes):
                raise ValueError(f"invalid workspace allocation: {a.name}")
            if a.name in self._index:
                raise ValueError(f"duplicate workspace allocation: {a.name}")
            self._index[a.name] = i
        # in order of first use only the values still live need comparing (a step of many
        # layers has hundreds of values and a handful live at a time)
        live: List[Allocation] = []
        for a in sorted(self.allocations, key=lambda x: x.first_use):
            live = [other for other in live if other.last_use >= a.first_use]
            for other in live:
                if a.offset < other.offset + other.bytes and other.offset < a.offset + a.bytes:
                    raise ValueError(f"overlapping live workspace allocations: {other.name} "
                                     f"and {a.name}")
            live.append(a)

    def __contains__(self, name: str) -> bool:
        return name in self._index

    def at(self, name: str) -> Allocation:
        try:
            return self.allocations[self._index[name]]
        except KeyError:
            raise KeyError(f"workspace allocation not found: {name}") from None

    # diagnostics of a plan
    def requested_bytes(self) -> int:
        return sum(a.bytes for a in self.allocations)

    def unaliased_bytes(self) -> int:
        """What the values would need one after the other, each aligned."""
        total = 0
        for a in self.allocations:
            total += (-total) % a.alignment + a.bytes
        return total

    def reused_bytes(self) -> int:
        return max(0, self.unaliased_bytes() - self.total_bytes)

    def slot_count(self) -> int:
        return len({a.offset for a in self.allocations})


class WorkspacePlanner:
    def __init__(self):
        self._requests: List[Allocation] = []
        self._names = set()

    def clear(self) -> None:
        self._requests.clear()
        self._names.clear()

    def add_request(self, name: str, nbytes: int, first_use: int, last_use: int,
                    alignment: int = 256) -> None:
        if not name:
            raise ValueError("a workspace request needs a name")
        if nbytes <= 0:
            raise ValueError(f"workspace request bytes must be positive for {name}")
        if first_use > last_use:
            raise ValueError(f"workspace request has an invalid lifetime for {name}")
        if not _power_of_two(alignment):
            raise ValueError(f"workspace alignment must be a power of two for {name}")
        if name in self._names:
            raise ValueError(f"duplicate workspace request: {name}")
        self._names.add(name)
        self._requests.append(Allocation(name, 0, int(nbytes), int(first_use), int(last_use),
                                         int(alignment)))

    def build(self) -> WorkspacePlan:
        ordered = sorted(self._requests, key=lambda r: (r.first_use, r.last_use, r.name))
        slots: List[List[int]] = []          # [offset, capacity, last use]
        allocations: List[Allocation] = []
        total = 0
        for request in ordered:
            best: Optional[List[int]] = None
            for slot in slots:
                # a last use at the new first use still overlaps
                if (slot[2] >= request.first_use or slot[1] < request.bytes
                        or slot[0] % request.alignment):
                    continue
                if best is None or (slot[1], slot[0]) < (best[1], best[0]):
                    best = slot
            if best is None:
                offset = (total + request.alignment - 1) // request.alignment * request.alignment
                best = [offset, request.bytes, request.last_use]
                slots.append(best)
                total = offset + request.bytes
            allocations.append(Allocation(request.name, best[0], request.bytes, request.first_use,
                                          request.last_use, request.alignment))
            best[2] = request.last_use
        return WorkspacePlan(allocations, total)
