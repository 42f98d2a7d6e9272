"""Gated feed-forward: down(silu(gate(x)) * up(x)).

runtime/include/execution/decoder.hpp:161-166 of the reference; gate and up are
two checkpoint matrices that become one [2I, H] matrix when the part is built.
"""
from __future__ import annotations

import torch

from ..csrc import lib
from ..weights.loader import ParamSpec
from .linear import Linear


class GatedMLP:
    @classmethod
    def parameters(cls, spec, hidden):
        return {
            "gate_proj.weight": ParamSpec((spec.intermediate_size, hidden)),
            "up_proj.weight": ParamSpec((spec.intermediate_size, hidden)),
            "down_proj.weight": ParamSpec((hidden, spec.intermediate_size)),
        }

    def __init__(self, spec, hidden, params, dtype, device):
        if spec.activation != "silu":
            raise ValueError(f"gated_mlp: activation '{spec.activation}' is not implemented")
        self.spec = spec
        self.gate_up = Linear(torch.cat([params["gate_proj.weight"], params["up_proj.weight"]],
                                        dim=0), dtype, device)
        self.down = Linear(params["down_proj.weight"], dtype, device)

    def forward(self, ctx, x):
        n = x.shape[0]
        gate_up = self.gate_up.forward(ctx, x, "mlp.gate_up")
        act = ctx.buffer("mlp.act", (n, self.spec.intermediate_size))
        lib.swiglu(gate_up, act)
        return self.down.forward(ctx, act, "mlp.down")
