"""Weights from safetensors, by tensor name.

Tensors keep the precision they are stored in when that is bfloat16 or 32-bit
float; 16-bit IEEE floats become bfloat16, 64-bit floats become 32-bit, and
integer tables become int32.  The parts decide later what they compute in.
A folder holds a single `model.safetensors` or a `model.safetensors.index.json` over
several files, which must lie inside the folder; nothing is ever downloaded (the same
rules as the reference's loader, frontend/checkpoint.py:58-105).  The container is read by
this package itself (`safetensors_file.py`): memory-mapped, tensor by tensor.
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


INDEX_FILE = "model.safetensors.index.json"
SINGLE_FILE = "model.safetensors"


def kept_precision(tensor: torch.Tensor) -> torch.Tensor:
    """bfloat16, float32 and int32 stay as they are; float16 becomes bfloat16, float64
    float32, every other integer type int32."""
    if tensor.dtype in (torch.bfloat16, torch.float32, torch.int32):
        return tensor
    if tensor.dtype == torch.float64:
        return tensor.to(torch.float32)
    if tensor.dtype.is_floating_point:
        return tensor.to(torch.bfloat16)
    return tensor.to(torch.int32)


def _file_inside(folder: Path, relative) -> Path:
    """The file `relative` names, which must lie inside `folder` (an index is data from
    outside: it must not be able to point anywhere else on the machine)."""
    if not isinstance(relative, str) or relative == "" or Path(relative).is_absolute():
        raise ValueError(f"a checkpoint file is named by a path relative to the model folder, "
                         f"got {relative!r}")
    target = (folder / relative).resolve()
    if folder not in target.parents:
        raise ValueError(f"every checkpoint file must lie inside the model folder; "
                         f"'{relative}' does not")
    if not target.is_file():
        raise FileNotFoundError(target)
    return target


def checkpoint_files(model_dir) -> Dict[Path, Optional[List[str]]]:
    """file -> the tensor names to take from it (None: all it holds).  A folder holds either
    an index over several files or the one file `model.safetensors`."""
    folder = Path(model_dir).resolve()
    index_path = folder / INDEX_FILE
    if not index_path.is_file():
        return {_file_inside(folder, SINGLE_FILE): None}
    listing = json.loads(index_path.read_text(encoding="utf-8"))
    placement = listing.get("weight_map") if isinstance(listing, dict) else None
    if not isinstance(placement, dict) or not placement:
        raise ValueError(f"{index_path} must hold a 'weight_map' from tensor names to files")
    files: Dict[Path, Optional[List[str]]] = {}
    for tensor_name, file_name in placement.items():
        files.setdefault(_file_inside(folder, file_name), []).append(tensor_name)
    return files


def read_tensors(model_dir) -> Dict[str, torch.Tensor]:
    """name -> tensor for everything the folder's checkpoint holds, in the kept precision.
    The tensors are views of the memory-mapped files (see `SafetensorsFile`) unless their
    type had to be converted, so asking for all of them reads next to nothing; nothing is
    ever downloaded.  EDGE_INFER_VERBOSE_WEIGHTS=1 lists them on standard output."""
    from .safetensors_file import SafetensorsFile

    chatty = os.environ.get("EDGE_INFER_VERBOSE_WEIGHTS") == "1"
    tensors: Dict[str, torch.Tensor] = {}
    for path, wanted in checkpoint_files(model_dir).items():
        container = SafetensorsFile(path)
        for name in (list(container.names()) if wanted is None else wanted):
            if name not in container:
                raise ValueError(f"the index places '{name}' in {path.name}, which does not "
                                 f"hold it")
            tensors[name] = kept_precision(container.tensor(name))
            if chatty:
                print(f"{path.name}: {name} {list(tensors[name].shape)} "
                      f"{str(tensors[name].dtype).replace('torch.', '')}")
    if not tensors:
        raise ValueError(f"the checkpoint in {model_dir} holds no tensors")
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
