"""Rotary position encoding: a float32 table of cosines and sines.

angle[p, i] = float(p) * (1 / theta^(2i / d)) with the frequency and the product
in float32, as the reference builds its table
(runtime/include/models/qwen3_model.hpp:410-436).  Its power is the C library's single
precision `pow`, which works in double precision inside and rounds the result once; the
same is done here (a float32 `pow` of another library may differ in the last bit, which
moves the angle of position 4,000 by 2e-4).  Cosine and sine are evaluated in float64 from
the float32 angle and rounded once.  Row p holds cos for the d/2 pairs, then sin; pairs are
(i, i + d/2).
"""
from __future__ import annotations

import torch


class RotaryTable:
    def __init__(self, spec, device):
        if spec.dim % 2:
            raise ValueError("rotary dimension must be even")
        self.spec = spec
        half = spec.dim // 2
        exponent = (2.0 * torch.arange(half, dtype=torch.float32)) / float(spec.dim)
        theta = torch.tensor(float(spec.theta), dtype=torch.float32).to(torch.float64)
        frequency = 1.0 / torch.pow(theta, exponent.to(torch.float64)).to(torch.float32)
        position = torch.arange(spec.max_positions, dtype=torch.float32)
        angle = (position[:, None] * frequency[None, :]).to(torch.float64)
        table = torch.cat([torch.cos(angle), torch.sin(angle)], dim=1).to(torch.float32)
        self.table = table.to(device).contiguous()

    @property
    def max_positions(self):
        return self.table.shape[0]


class NoPosition:
    """Mixers that take no position encoding get a table of None."""
    def __init__(self, spec, device):
        self.spec = spec
        self.table = None
        self.max_positions = None
