"""Laying out the buffers of a step in one arena: buffers that are never live at the same
time share bytes.

A step is a sequence of ticks.  Each buffer has a `Lifetime`: the tick at which it is first
written (`born`) and the last tick at which it is read (`dies`).  `lay_out` walks the
lifetimes in birth order and keeps a list of regions of the arena; a buffer moves into the
tightest region whose previous tenant is dead (died strictly before the newcomer is born:
at the same tick a kernel may still read the one while it writes the other), that is large
enough and suitably aligned; if there is none the arena grows by a new region.  Nothing is
allocated here: the result says where in an arena of `arena_bytes` each buffer lies.

The reference plans its decoder buffers offline in the same way and this module answers
its planner's test vectors the same way (core/include/execution/workspace_plan.hpp:138-252,
operators/tests/decode_workspace_plan_test.cpp:16-60); the lifetimes here are not declared
by hand but recorded from a step that ran (`parts.base.Workspace`).
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Dict, Iterable, List

DEFAULT_ALIGNMENT = 256


@dataclass(frozen=True)
class Lifetime:
    """A buffer's need: `nbytes` from tick `born` through tick `dies`, at an address that is
    a multiple of `alignment` (a power of two)."""
    name: str
    nbytes: int
    born: int
    dies: int
    alignment: int = DEFAULT_ALIGNMENT

    def check(self) -> None:
        if not self.name:
            raise ValueError("a buffer needs a name")
        if self.nbytes <= 0:
            raise ValueError(f"buffer '{self.name}': its size must be positive")
        if self.born > self.dies:
            raise ValueError(f"buffer '{self.name}': it dies before it is born")
        if self.alignment <= 0 or self.alignment & (self.alignment - 1):
            raise ValueError(f"buffer '{self.name}': the alignment must be a power of two")


@dataclass(frozen=True)
class Placement:
    """Where a buffer lies in the arena."""
    need: Lifetime
    offset: int

    @property
    def end(self) -> int:
        return self.offset + self.need.nbytes


class ArenaLayout:
    """Placements by buffer name.  Construction proves the layout: every buffer inside the
    arena and aligned, and no two buffers that are live at the same tick on the same bytes."""

    def __init__(self, placements: Iterable[Placement], arena_bytes: int):
        self.arena_bytes = int(arena_bytes)
        self._by_name: Dict[str, Placement] = {}
        for placement in placements:
            need = placement.need
            need.check()
            if need.name in self._by_name:
                raise ValueError(f"buffer '{need.name}' is placed twice")
            if placement.offset < 0 or placement.end > self.arena_bytes:
                raise ValueError(f"buffer '{need.name}' lies outside the arena")
            if placement.offset % need.alignment:
                raise ValueError(f"buffer '{need.name}' is misaligned")
            self._by_name[need.name] = placement
        # sweep in birth order; only buffers that have not died yet can collide
        living: List[Placement] = []
        for placement in sorted(self._by_name.values(), key=lambda p: p.need.born):
            living = [other for other in living if other.need.dies >= placement.need.born]
            for other in living:
                if placement.offset < other.end and other.offset < placement.end:
                    raise ValueError(f"buffers '{other.need.name}' and '{placement.need.name}' "
                                     f"are live together on the same bytes")
            living.append(placement)

    def __contains__(self, name: str) -> bool:
        return name in self._by_name

    def __len__(self) -> int:
        return len(self._by_name)

    def names(self):
        return list(self._by_name)

    def offset(self, name: str) -> int:
        try:
            return self._by_name[name].offset
        except KeyError:
            raise KeyError(f"the layout holds no buffer '{name}'") from None

    # what sharing buys
    def bytes_asked(self) -> int:
        """The sum of the buffers' sizes."""
        return sum(p.need.nbytes for p in self._by_name.values())

    def bytes_without_sharing(self) -> int:
        """The arena that the same buffers would need side by side, each aligned."""
        total = 0
        for placement in self._by_name.values():
            total += (-total) % placement.need.alignment + placement.need.nbytes
        return total

    def bytes_saved(self) -> int:
        return max(0, self.bytes_without_sharing() - self.arena_bytes)

    def regions(self) -> int:
        """Distinct places in use: the fewer for the same buffers, the more sharing."""
        return len({p.offset for p in self._by_name.values()})


def lay_out(lifetimes: Iterable[Lifetime]) -> ArenaLayout:
    needs = list(lifetimes)
    seen = set()
    for need in needs:
        need.check()
        if need.name in seen:
            raise ValueError(f"buffer '{need.name}' is asked for twice")
        seen.add(need.name)
    needs.sort(key=lambda need: (need.born, need.dies, need.name))
    regions: List[List[int]] = []          # [offset, size, tick at which its tenant dies]
    placements: List[Placement] = []
    arena = 0
    for need in needs:
        home = None
        for region in regions:
            offset, size, free_after = region
            if free_after >= need.born or size < need.nbytes or offset % need.alignment:
                continue
            if home is None or (size, offset) < (home[1], home[0]):
                home = region
        if home is None:
            offset = -(-arena // need.alignment) * need.alignment
            home = [offset, need.nbytes, need.dies]
            regions.append(home)
            arena = offset + need.nbytes
        home[2] = need.dies
        placements.append(Placement(need, home[0]))
    return ArenaLayout(placements, arena)
