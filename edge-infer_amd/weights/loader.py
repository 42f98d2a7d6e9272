"""Weights from safetensors, by tensor name.

Tensors keep the precision they are stored in when that is bfloat16 or 32-bit
float; 16-bit IEEE floats become bfloat16, 64-bit floats become 32-bit, and
integer tables become int32.  The parts decide later what they compute in.
File handling follows frontend/checkpoint.py:58-105 of the reference: a single
`model.safetensors` or a `model.safetensors.index.json` whose shards must stay
inside the model folder; nothing is ever downloaded.
"""
from __future__ import annotations

import json
import os
from dataclasses import dataclass, field
from pathlib import Path
from typing import Dict, List, Mapping, Optional, Tuple

import torch


@dataclass(frozen=True)
class ParamSpec:
    """One parameter a part expects.  `init` chooses the random-weights law:
    "normal" (N(0, 0.02)) for matrices and tables, "norm" (1 + U(-0.1, 0.1)).
    `optional`: taken when the checkpoint holds it, no error when it does not (the
    reference's optional projection biases, runtime/include/models/qwen3_model.hpp:371-403)."""
    shape: Tuple[int, ...]
    init: str = "normal"
    optional: bool = False


@dataclass
class WeightsError(ValueError):
    """All that is wrong with a checkpoint, in one message."""
    missing: List[str] = field(default_factory=list)
    unexpected: List[str] = field(default_factory=list)
    wrong_shape: List[Tuple[str, Tuple[int, ...], Tuple[int, ...]]] = field(default_factory=list)
    duplicate: List[str] = field(default_factory=list)   # stored under two of its names

    def __str__(self) -> str:
        lines = ["checkpoint does not match the model:"]
        if self.missing:
            lines.append(f"  missing tensors ({len(self.missing)}): " + ", ".join(self.missing))
        if self.unexpected:
            lines.append(f"  unexpected tensors ({len(self.unexpected)}): "
                         + ", ".join(self.unexpected))
        if self.wrong_shape:
            lines.append(f"  wrong shapes ({len(self.wrong_shape)}): " + ", ".join(
                f"{name} expected {list(want)} got {list(got)}"
                for name, want, got in self.wrong_shape))
        if self.duplicate:
            lines.append(f"  stored twice, under a second name as well ({len(self.duplicate)}): "
                         + ", ".join(self.duplicate))
        return "\n".join(lines)


def _shard_path(root: Path, name) -> Path:
    if not isinstance(name, str) or not name or Path(name).is_absolute():
        raise ValueError("checkpoint shard names must be relative paths")
    path = (root / name).resolve()
    try:
        path.relative_to(root)
    except ValueError as error:
        raise ValueError("checkpoint shards must stay inside the model folder") from error
    if not path.is_file():
        raise FileNotFoundError(path)
    return path


def _stored_precision(tensor: torch.Tensor) -> torch.Tensor:
    if tensor.dtype in (torch.bfloat16, torch.float32, torch.int32):
        return tensor
    if tensor.dtype == torch.float16:
        return tensor.to(torch.bfloat16)
    if tensor.dtype == torch.float64:
        return tensor.to(torch.float32)
    if not tensor.dtype.is_floating_point:
        return tensor.to(torch.int32)
    return tensor.to(torch.bfloat16)


def read_tensors(model_dir) -> Dict[str, torch.Tensor]:
    """Every tensor of the folder's safetensors file(s), on the host."""
    from safetensors import safe_open

    root = Path(model_dir).resolve()
    index_path = root / "model.safetensors.index.json"
    if index_path.is_file():
        with index_path.open(encoding="utf-8") as source:
            index = json.load(source)
        weight_map = index.get("weight_map") if isinstance(index, dict) else None
        if not isinstance(weight_map, dict) or not weight_map:
            raise ValueError("the safetensors index must hold a nonempty weight_map")
        shards: Dict[Path, Optional[List[str]]] = {}
        for name, shard in weight_map.items():
            shards.setdefault(_shard_path(root, shard), []).append(name)
    else:
        shards = {_shard_path(root, "model.safetensors"): None}
    # EDGE_INFER_VERBOSE_WEIGHTS=1 lists what is read, as in frontend/checkpoint.py:88-99
    verbose = os.environ.get("EDGE_INFER_VERBOSE_WEIGHTS") == "1"
    tensors: Dict[str, torch.Tensor] = {}
    for path, names in shards.items():
        with safe_open(str(path), framework="pt", device="cpu") as source:
            for name in (source.keys() if names is None else names):
                tensors[name] = _stored_precision(source.get_tensor(name))
                if verbose:
                    print(f"Loaded {name}: {tuple(tensors[name].shape)}, {tensors[name].dtype}")
    if not tensors:
        raise ValueError("the checkpoint holds no tensors")
    return tensors


def match_parameters(expected: Mapping[str, Tuple[str, ParamSpec]],
                     tensors: Mapping[str, torch.Tensor],
                     optional: Mapping[str, str] = (),
                     aliases: Mapping[str, str] = ()) -> Dict[str, torch.Tensor]:
    """Map model parameters to checkpoint tensors.

    `expected`: parameter path -> (checkpoint name, spec).  `optional`: parameter
    path -> parameter path it may be taken from when its own tensor is absent
    (a tied output head).  `aliases`: other checkpoint names for the same
    tensor.  Raises one `WeightsError` that lists every missing tensor, every
    tensor the model has no use for, every wrong shape, and every tensor that is stored
    under two of its names.
    """
    optional = dict(optional)
    available = {}
    error = WeightsError()
    for name, tensor in tensors.items():
        canonical = dict(aliases).get(name, name)
        if canonical in available:   # bindings/python/include/decoder_weight_mapper.hpp:173
            error.duplicate.append(canonical)
        available[canonical] = tensor
    result: Dict[str, torch.Tensor] = {}
    used = set()
    for parameter, (name, spec) in expected.items():
        if name not in available:
            if parameter in optional or spec.optional:
                continue
            error.missing.append(name)
            continue
        used.add(name)
        tensor = available[name]
        if tuple(tensor.shape) != tuple(spec.shape):
            error.wrong_shape.append((name, tuple(spec.shape), tuple(tensor.shape)))
            continue
        result[parameter] = tensor
    for parameter, source in optional.items():
        if parameter not in result and expected[parameter][0] not in available:
            if source in result:
                result[parameter] = result[source]
    error.unexpected = sorted(set(available) - used)
    if error.missing or error.unexpected or error.wrong_shape or error.duplicate:
        raise error
    return result
