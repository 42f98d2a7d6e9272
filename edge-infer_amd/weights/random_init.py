"""Random-weights mode: a model folder (config.json, model.safetensors) from a
configuration and a seed.  Matrices and tables are N(0, 0.02), norm weights
1 + U(-0.1, 0.1), stored in bfloat16; optional parameters (biases) are left out unless
asked for, and then N(0, 0.02) too.  The reference has no such mode (its tests
build closed-form weights, runtime/tests/qwen3_session_test.cpp:124-172)."""
from __future__ import annotations

import json
from pathlib import Path
from typing import Dict, Mapping, Tuple

import torch

from .loader import ParamSpec


def random_tensor(spec: ParamSpec, generator: torch.Generator, device="cpu",
                  dtype=torch.bfloat16) -> torch.Tensor:
    shape = tuple(spec.shape)
    if spec.init == "normal":
        value = torch.randn(shape, generator=generator, device=device, dtype=torch.float32) * 0.02
    elif spec.init == "norm":
        value = 1.0 + (torch.rand(shape, generator=generator, device=device,
                                  dtype=torch.float32) * 0.2 - 0.1)
    else:
        raise ValueError(f"unknown initialisation '{spec.init}'")
    return value.to(dtype)


def random_parameters(expected: Mapping[str, Tuple[str, ParamSpec]], seed: int, device="cpu",
                      dtype=torch.bfloat16, skip=(), biases=False) -> Dict[str, torch.Tensor]:
    """parameter path -> tensor, drawn in the order of `expected`; optional parameters
    only with `biases`."""
    generator = torch.Generator(device=device)
    generator.manual_seed(int(seed))
    return {parameter: random_tensor(spec, generator, device, dtype)
            for parameter, (_, spec) in expected.items()
            if parameter not in skip and (biases or not spec.optional)}


def write_model_folder(path, config, seed: int, biases: bool = False) -> Path:
    """Write config.json and model.safetensors for `config` (an architecture's
    typed configuration) with weights from `seed`.  A tied head is not stored.
    `biases`: every projection and the head get a bias as well."""
    from safetensors.torch import save_file
    from ..engine.model import expected_parameters

    path = Path(path)
    path.mkdir(parents=True, exist_ok=True)
    spec = config.model_spec()
    expected = expected_parameters(spec, config.checkpoint_name)
    skip = ("head.weight",) if spec.tie_word_embeddings else ()
    parameters = random_parameters(expected, seed, skip=skip, biases=biases)
    tensors = {expected[parameter][0]: tensor.contiguous()
               for parameter, tensor in parameters.items()}
    (path / "config.json").write_text(json.dumps(config.to_dict(), indent=2) + "\n")
    save_file(tensors, str(path / "model.safetensors"), metadata={"format": "pt"})
    return path
