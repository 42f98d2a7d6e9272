"""edge-infer for AMD MI355X: a small Qwen3-dense generation library.

    model = load_model("/path/to/folder", dtype="bfloat16")     # config.json + safetensors
    session = Session(model, max_tokens=4096)
    slot = session.begin()
    logits = session.step([(slot, [5, 17, 3], [2])])            # float32 [1, vocab]

Importing the package needs no GPU; building a model or a session does.
"""
from __future__ import annotations

from . import config, parts  # registers the built-in architecture and parts
from .config import Qwen3Config, read_config, register_architecture
from .weights import WeightsError, write_model_folder

__version__ = "0.1.0"


def require_gpu(device="cuda"):
    import torch
    if not torch.cuda.is_available():
        raise RuntimeError("edge-infer needs an AMD GPU (gfx950): torch.cuda.is_available() is "
                           "False and there is no CPU implementation to fall back to")
    return torch.device(device)


def build_model(entry, cfg, tensors, dtype="bfloat16", device="cuda"):
    """The model of a registered architecture (`entry`, its typed configuration `cfg`) from
    checkpoint tensors by name: the one assembly behind `load_model` and `api.Model`."""
    from .engine.model import DecoderModel, expected_parameters
    from .weights import match_parameters

    device = require_gpu(device)
    spec = cfg.model_spec()
    expected = expected_parameters(spec, cfg.checkpoint_name)
    optional = {"head.weight": "embed.weight"} if spec.tie_word_embeddings else {}
    params = match_parameters(expected, tensors, optional=optional,
                              aliases=getattr(cfg, "checkpoint_aliases", {}))
    factory = entry.model_factory or DecoderModel
    model = factory(spec, params, dtype, device)
    model.config = cfg
    return model


def load_model(model_dir, dtype="bfloat16", device="cuda"):
    """Build the model that the folder's config.json names, with its weights."""
    from .weights import read_tensors

    entry, cfg, _ = read_config(model_dir)
    return build_model(entry, cfg, read_tensors(model_dir), dtype, device)


def random_model(cfg, seed, dtype="bfloat16", device="cuda", biases=False):
    """A model of configuration `cfg` with random weights drawn on the device (`biases`:
    with the optional bias of every projection and of the head)."""
    from .config.registry import architecture_entry
    from .engine.model import DecoderModel, expected_parameters
    from .weights import random_parameters

    device = require_gpu(device)
    spec = cfg.model_spec()
    expected = expected_parameters(spec, cfg.checkpoint_name)
    skip = ("head.weight",) if spec.tie_word_embeddings else ()
    params = random_parameters(expected, seed, device=device, skip=skip, biases=biases)
    # the model class is the registry's, as for a model read from a folder
    entry = architecture_entry(getattr(cfg, "architecture", spec.architecture))
    factory = (entry.model_factory if entry is not None else None) or DecoderModel
    model = factory(spec, params, dtype, device)
    model.config = cfg
    return model


def __getattr__(name):
    if name == "Session":
        from .engine.session import Session
        return Session
    if name in ("Model", "generate", "SamplingParams", "Generator"):
        from . import api
        return getattr(api, name)
    raise AttributeError(name)
