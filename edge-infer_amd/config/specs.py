"""Architecture-independent description of a decoder: what the engine builds from.

An architecture's own configuration (for example `Qwen3Config`) is translated
into a `ModelSpec`: a tuple of `LayerSpec`s, each naming its block arrangement,
norm, mixer and feed-forward with every size and constant as a field, plus a
`schedule` that says in which order layers run and which cache each run uses.
Parts are selected by the `kind` strings through `parts.registry`; nothing in
this file knows a model family.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Optional, Tuple


@dataclass(frozen=True)
class NormSpec:
    kind: str = "rmsnorm"
    eps: float = 1e-6


@dataclass(frozen=True)
class PositionSpec:
    """Position encoding of a mixer.  kind "rope": rotate-half pairs (i, i+dim/2)
    with angle = position / theta^(2i/dim); kind "none": no encoding."""
    kind: str = "rope"
    theta: float = 10000.0
    dim: int = 0
    max_positions: int = 0


@dataclass(frozen=True)
class AttentionSpec:
    """Causal grouped-query attention over a key/value cache."""
    kind: str = "attention"
    n_heads: int = 0
    n_kv_heads: int = 0
    head_dim: int = 0
    qk_norm: bool = False          # per-head RMSNorm of q and k before the rotation
    qk_norm_eps: float = 1e-6
    window: Optional[int] = None   # None: every earlier key; w: the last w keys
    scale: Optional[float] = None  # None: 1/sqrt(head_dim)
    position: PositionSpec = field(default_factory=PositionSpec)

    @property
    def q_width(self) -> int:
        return self.n_heads * self.head_dim

    @property
    def kv_width(self) -> int:
        return self.n_kv_heads * self.head_dim


@dataclass(frozen=True)
class GatedMLPSpec:
    """down(act(gate(x)) * up(x))."""
    kind: str = "gated_mlp"
    intermediate_size: int = 0
    activation: str = "silu"


@dataclass(frozen=True)
class LayerSpec:
    block: str            # arrangement, e.g. "prenorm"
    norm: NormSpec
    mixer: object         # a spec with a .kind (AttentionSpec, or one a test registers)
    feed_forward: object  # a spec with a .kind (GatedMLPSpec, ...)


@dataclass(frozen=True)
class ScheduleEntry:
    """One run of a layer.  `cache` is the id of the cache entry the mixer uses;
    `writes_cache` False means it only reads an entry that another run wrote."""
    layer: int
    cache: int
    writes_cache: bool = True


@dataclass(frozen=True)
class ModelSpec:
    architecture: str
    vocab_size: int
    hidden_size: int
    layers: Tuple[LayerSpec, ...]
    schedule: Tuple[ScheduleEntry, ...]
    final_norm: NormSpec
    tie_word_embeddings: bool
    max_position_embeddings: int
    bos_token_id: int
    eos_token_id: int

    def validate(self) -> None:
        if not self.layers or not self.schedule:
            raise ValueError("a model needs at least one layer and one schedule entry")
        writers = {}
        for entry in self.schedule:
            if not 0 <= entry.layer < len(self.layers):
                raise ValueError(f"schedule names layer {entry.layer} of {len(self.layers)}")
            if entry.writes_cache:
                if entry.cache in writers:
                    raise ValueError(f"cache entry {entry.cache} has two writers")
                writers[entry.cache] = entry.layer
        seen = set()
        for entry in self.schedule:
            if entry.writes_cache:
                seen.add(entry.cache)
            elif entry.cache not in seen:
                raise ValueError(
                    f"layer {entry.layer} reads cache entry {entry.cache} before it is written")


def default_schedule(n_layers: int) -> Tuple[ScheduleEntry, ...]:
    """Every layer once, in order, each with a cache entry of its own."""
    return tuple(ScheduleEntry(layer=i, cache=i) for i in range(n_layers))
