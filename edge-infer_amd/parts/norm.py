"""RMSNorm fused with the residual addition that precedes it.

y = x * rsqrt(mean(x^2) + eps) * w, all in float32, rounded once to the storage
type (the reference's float32 path, operators/src/cuda/rms_norm_cuda.cu:99-100;
its bfloat16 path rounds twice, :91-98, which this implementation does not copy).
The weight is kept in float32 whatever it was stored in.
"""
from __future__ import annotations

import torch

from ..csrc import lib
from ..weights.loader import ParamSpec


class RMSNorm:
    capture_safe = True      # only capturable kernels, no allocation per step

    @classmethod
    def kernel_libraries(cls, spec, dtype):
        return ("rowwise",)

    @classmethod
    def parameters(cls, spec, width):
        return {"weight": ParamSpec((width,), init="norm")}

    def __init__(self, spec, width, params, dtype, device):
        self.eps = float(spec.eps)
        self.width = width
        self.weight = params["weight"].to(device=device, dtype=torch.float32).contiguous()

    def add_norm(self, ctx, residual, delta, out_name, rows=None, write_residual=True):
        """residual += delta (all splits); returns rmsnorm(residual)[rows] * weight in
        the step's storage type."""
        n = residual.shape[0] if rows is None else rows.numel()
        out = ctx.buffer(out_name, (n, self.width))
        lib.add_rmsnorm(residual, delta, self.weight, self.eps, out, rows=rows,
                        write_residual=write_residual)
        return out
