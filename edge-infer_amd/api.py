"""Python entry point in the manner of the reference's `model_bridge`
(bindings/python/model_bridge.cpp:245-294, docs/python-api.md):

    config, weights, model_type = load_checkpoint(path, "qwen3_bf16")
    model = Model(config, weights, model_type, device="cuda")
    session = model.new_session(capacity=1024)
    session.generate(prompt_ids, tokens.append, max_length=len(prompt_ids) + 32, top_k=1)
    session.reset()

`Model` prepares weights and holds no cache; sessions share its weights and own
their caches.  Beyond the reference, a session can serve a batch of prompts
(`new_session(max_batch=8)`, `session.generate_batch`) and exposes the step function
(`session.step`).  Model types: "qwen3_bf16" (the reference's name) and
"qwen3_fp32" for the true 32-bit path.

The reference's procedural wrappers over one implicit session are here too
(model_bridge.cpp:159-215,274-283): `init_model`, `generate_text_stream`,
`set_default_device`, `get_default_device`, `is_cuda_available`.
"""
from __future__ import annotations

import json
import sys
from pathlib import Path
from typing import Mapping, Optional

import torch

from . import build_model, require_gpu
from .config import resolve_architecture
from .engine.generate import generate  # noqa: F401  (re-exported)
from .engine.session import Session
from .sampling.params import SamplingParams  # noqa: F401
from .weights import read_tensors

MODEL_TYPES = {"qwen3_bf16": "bfloat16", "qwen3_fp32": "float32"}
DEFAULT_CAPACITY = 4096   # bindings/python/model_bridge.cpp:135-141: min(4096, model limit)


def load_checkpoint(model_path, model_type="qwen3_bf16"):
    """What `Model` takes, from a local folder: (config.json as a dict, {tensor name:
    tensor}, model type).  The reference's frontend hands its bridge the same three things
    (frontend/checkpoint.py:58-105); the tensors here are views of the mapped files."""
    _known_type(model_type)
    folder = Path(model_path)
    config = json.loads((folder / "config.json").read_text(encoding="utf-8"))
    if not isinstance(config, dict):
        raise ValueError(f"{folder / 'config.json'} must hold a JSON object")
    return config, read_tensors(folder), model_type


def _known_type(model_type) -> str:
    """The compute type a model type stands for."""
    try:
        return MODEL_TYPES[model_type]
    except (KeyError, TypeError):
        raise ValueError(f"unsupported model type {model_type!r}; "
                         f"known: {sorted(MODEL_TYPES)}") from None


class Model:
    def __init__(self, config: Mapping, weights: Mapping[str, torch.Tensor],
                 model_type: str = "qwen3_bf16", device: Optional[str] = None):
        dtype = _known_type(model_type)
        if device not in (None, "cuda") and not str(device).startswith("cuda"):
            raise ValueError("this library runs on the GPU only (device 'cuda')")
        self._device = require_gpu(device or "cuda")
        entry = resolve_architecture(config)
        self.config = entry.config_class.from_dict(config)
        self.decoder = build_model(entry, self.config, weights, dtype, self._device)
        self.model_type = model_type

    @classmethod
    def from_pretrained(cls, model_path, model_type="qwen3_bf16", device=None) -> "Model":
        config, weights, model_type = load_checkpoint(model_path, model_type)
        return cls(config, weights, model_type, device)

    @property
    def device(self) -> str:
        return str(self._device)

    @property
    def max_context_length(self) -> int:
        return self.decoder.max_positions()

    def new_session(self, capacity: Optional[int] = None, max_batch: int = 1,
                    seed: int = 0) -> Session:
        """An independent session whose sequences hold up to `capacity` tokens each
        (default min(4096, model limit)), `max_batch` of them at a time."""
        limit = self.max_context_length
        if capacity is None:
            capacity = min(DEFAULT_CAPACITY, limit)
        if isinstance(capacity, bool) or not isinstance(capacity, int) or not 1 <= capacity <= limit:
            raise ValueError(f"capacity must lie in 1..{limit}, got {capacity!r}")
        if max_batch < 1:
            raise ValueError("max_batch must be positive")
        pages_each = (capacity + 63) // 64
        return Session(self.decoder, max_tokens=pages_each * 64 * max_batch, max_seqs=max_batch,
                       max_seq_tokens=capacity, seed=seed)


def is_gpu_available() -> bool:
    return torch.cuda.is_available()


# -- the procedural interface: one implicit model and session ---------------------------
_compat = {"model": None, "session": None, "busy": False}


class _Operation:
    """One call of the procedural interface at a time: a callback that calls back in is an
    error, as in the reference (model_bridge.cpp:165-168)."""

    def __enter__(self):
        if _compat["busy"]:
            raise RuntimeError("the runtime is busy with another operation")
        _compat["busy"] = True

    def __exit__(self, *exc):
        _compat["busy"] = False
        return False


def init_model(config: Mapping, weights: Mapping[str, torch.Tensor],
               model_type: str = "qwen3_bf16") -> bool:
    """Replace the implicit model and its session (default capacity); on failure the
    previous ones stay, the reason goes to stderr and False comes back."""
    with _Operation():
        try:
            model = Model(config, weights, model_type)
            session = model.new_session()
        except Exception as error:                      # the reference catches everything here
            print(f"Error initializing model: {error}", file=sys.stderr)
            return False
        _compat["model"], _compat["session"] = model, session
        return True


def generate_text_stream(input_ids, callback, max_length: int = 100, temperature: float = 1.0,
                         top_p: float = 0.9, top_k: int = 50) -> None:
    """`Session.generate` on the implicit session (note the other default of top_k)."""
    with _Operation():
        if _compat["session"] is None:
            raise RuntimeError("Model not initialized")
        _compat["session"].generate(list(input_ids), callback, max_length=max_length,
                                    temperature=temperature, top_p=top_p, top_k=top_k)


def set_default_device(device: str) -> bool:
    """Only "cuda" can be the default here: there is no CPU path."""
    with _Operation():
        try:
            if str(device) != "cuda" and not str(device).startswith("cuda:"):
                raise ValueError(f"unsupported device '{device}': this library runs on the GPU only")
            if not torch.cuda.is_available():
                raise RuntimeError("cuda requested but no GPU is available")
            return True
        except Exception as error:
            print(f"Error setting default device: {error}", file=sys.stderr)
            return False


def get_default_device() -> str:
    return "cuda"


def is_cuda_available() -> bool:
    """The reference's name; `is_gpu_available` is the same."""
    return is_gpu_available()
