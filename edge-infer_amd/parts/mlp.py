"""Gated feed-forward: down(silu(gate(x)) * up(x)).

runtime/include/execution/decoder.hpp:161-166 of the reference; gate and up are
two checkpoint matrices that become one [2I, H] matrix when the part is built: in strips
of 16 rows, the gate rows of 16 outputs followed by their up rows (when I is a multiple of
16; else all gate rows, then all up rows).  A wave of the few-rows kernel owns 16 rows, so
neighbouring waves hold a strip's gate and up sums and the kernel can write
silu(gate) * up itself; otherwise the activation kernel reads the same layout.
Optional biases (runtime/include/models/qwen3_model.hpp:396-403) follow their rows.
"""
from __future__ import annotations

import torch

from ..csrc import lib
from ..weights.loader import ParamSpec
from .linear import Linear


class GatedMLP:
    @property
    def capture_safe(self):
        """Only capturable kernels and no allocation per step, as long as its products do."""
        return self.gate_up.capture_safe and self.down.capture_safe

    @property
    def capture_rows(self):
        return min(self.gate_up.capture_rows, self.down.capture_rows)

    @classmethod
    def kernel_libraries(cls, spec, dtype):
        return ("rowwise", *Linear.kernel_libraries(dtype))

    @classmethod
    def parameters(cls, spec, hidden):
        return {
            "gate_proj.weight": ParamSpec((spec.intermediate_size, hidden)),
            "up_proj.weight": ParamSpec((spec.intermediate_size, hidden)),
            "down_proj.weight": ParamSpec((hidden, spec.intermediate_size)),
            "gate_proj.bias": ParamSpec((spec.intermediate_size,), optional=True),
            "up_proj.bias": ParamSpec((spec.intermediate_size,), optional=True),
            "down_proj.bias": ParamSpec((hidden,), optional=True),
        }

    def __init__(self, spec, hidden, params, dtype, device):
        if spec.activation != "silu":
            raise ValueError(f"gated_mlp: activation '{spec.activation}' is not implemented")
        self.spec = spec
        gate, up = params["gate_proj.weight"], params["up_proj.weight"]
        inter = spec.intermediate_size
        self.strip = lib.GATE_STRIP if inter % lib.GATE_STRIP == 0 else 0
        if self.strip:
            both = torch.stack([gate.reshape(inter // self.strip, self.strip, hidden),
                                up.reshape(inter // self.strip, self.strip, hidden)], dim=1)
            both = both.reshape(2 * inter, hidden)
        else:
            both = torch.cat([gate, up], dim=0)
        both_bias = None
        if "gate_proj.bias" in params or "up_proj.bias" in params:   # an absent one is zero
            zero = gate.new_zeros(inter)
            gate_bias = params.get("gate_proj.bias", zero)
            up_bias = params.get("up_proj.bias", zero)
            if self.strip:    # the same interleaving as the rows
                both_bias = torch.stack([gate_bias.reshape(-1, self.strip),
                                         up_bias.reshape(-1, self.strip)], dim=1).reshape(-1)
            else:
                both_bias = torch.cat([gate_bias, up_bias])
        self.gate_up = Linear(both, dtype, device, bias=both_bias)
        self.down = Linear(params["down_proj.weight"], dtype, device,
                           bias=params.get("down_proj.bias"))

    def forward(self, ctx, x):
        n = x.shape[0]
        act = self.gate_up.forward_gated(ctx, x, "mlp.act") if self.strip else None
        if act is None:
            gate_up = self.gate_up.forward(ctx, x, "mlp.gate_up")
            act = ctx.buffer("mlp.act", (n, self.spec.intermediate_size))
            lib.swiglu(gate_up, act, self.strip)
            ctx.release(gate_up)
        out = self.down.forward(ctx, act, "mlp.down")
        ctx.release(act)
        return out
