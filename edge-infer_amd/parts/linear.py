"""y = x . W^T for a checkpoint matrix kept in its stored [out, in] layout.

float32: the hand-written float32 kernel (no reduced-precision matrix mode).
bfloat16: for up to `SKINNY_ROWS` rows the hand-written weight-streaming MFMA
kernel, which returns float32 partial sums [slices, rows, out] that the consuming
kernel adds up while it reads them; for more rows the library matrix product (the reference multiplies
through cuBLAS as well, operators/src/cuda/execution.cu:299-324).

The few-rows kernel reads a second copy of the weight in its streaming layout (tiles in
the order in which the matrix cores take them, see `lib.pack_weight`), made when the
weight is loaded: decode is bound by how fast the weights can be read, and the
contiguous copy reads about a fifth faster than rows that lie a power of two apart.  It
doubles the memory of the linear weights; EDGE_INFER_STREAM_COPY=0 keeps only the stored
layout and lets the kernel read that.

An optional bias [out] enters the sum before the one rounding, as in the reference
(operators/src/cuda/execution.cu:307-317 fills the product's accumulator with it): as one
more float32 slice beside the few-rows kernel's, as the library product's addend, or added
to the float32 product.
"""
from __future__ import annotations

import os

import torch

from ..csrc import lib

SKINNY_ROWS = lib.SKINNY_ROWS
STREAM_COPY = os.environ.get("EDGE_INFER_STREAM_COPY", "1") != "0"
# The gated product does not slice K.  Where the planner would slice, one kernel still beats
# the sliced product plus the activation kernel while the matrix is small enough for a launch
# to weigh as much as the slicing gains (measured at 1 to 32 rows: 12.6 MB 5.6 against 7.2 us,
# 100 MB 17.2 against 20.9, 357 MB 62.2 against 61.2, 524 MB 90.4 against 83.9).
GATED_UNSLICED_BYTES = 200 * 1000 * 1000


class Linear:
    @staticmethod
    def kernel_libraries(dtype):
        """The kernel libraries a product in `dtype` runs."""
        return ("gemm_bf16", "rowwise") if dtype == torch.bfloat16 else ("gemm_f32", "rowwise")

    def __init__(self, weight: torch.Tensor, dtype, device, bias: torch.Tensor = None):
        if weight.dim() != 2:
            raise ValueError("a linear weight must be a matrix [out, in]")
        self.weight = weight.to(device=device, dtype=dtype).contiguous()
        self.out_features, self.in_features = self.weight.shape
        self.dtype = dtype
        self.bias = self.bias_f32 = None
        if bias is not None:
            if tuple(bias.shape) != (self.out_features,):
                raise ValueError(f"a linear bias must be [{self.out_features}], "
                                 f"got {list(bias.shape)}")
            self.bias = bias.to(device=device, dtype=dtype).contiguous()
            self.bias_f32 = self.bias.to(torch.float32)
        self.packed = None
        if dtype == torch.bfloat16 and STREAM_COPY and self.in_features % 8 == 0:
            self.packed = lib.pack_weight(self.weight)

    @property
    def capture_safe(self) -> bool:
        """Whether a step of at most `capture_rows` rows launches nothing but this library's
        kernels here (the library's products may record memset nodes, which are not replayed
        reliably from a graph)."""
        return self.dtype == torch.float32 or self.in_features % 8 == 0

    @property
    def capture_rows(self) -> int:
        """Most rows of a step for which `capture_safe` holds."""
        return (1 << 30) if self.dtype == torch.float32 else SKINNY_ROWS

    def _few_rows(self, x: torch.Tensor, out: torch.Tensor) -> None:
        if self.packed is not None:
            lib.gemm_bf16_skinny_packed(x, self.packed, self.out_features, out)
        else:
            lib.gemm_bf16_skinny(x, self.weight, out)

    def forward(self, ctx, x: torch.Tensor, out_name: str) -> torch.Tensor:
        """x [N, in] of the step's storage type -> [N, out] in the storage type, or float32
        partial sums [slices, N, out] when the few-rows kernel ran; the result lives in the
        workspace buffer `out_name`."""
        rows = x.shape[0]
        if self.dtype == torch.float32:
            out = ctx.buffer(out_name, (rows, self.out_features), torch.float32)
            lib.gemm_f32(x, self.weight, out)
            if self.bias is not None:
                lib.bias_rows(self.bias_f32, out, accumulate=True)
            return out
        if lib.skinny_gemm_ok(rows, self.in_features):
            splits = lib.skinny_gemm_splits(rows, self.out_features, self.in_features)
            extra = 0 if self.bias is None else 1
            out = ctx.buffer(out_name + ".f32", (splits + extra, rows, self.out_features),
                             torch.float32)
            self._few_rows(x, out[:splits])
            if extra:
                lib.bias_rows(self.bias_f32, out[splits], accumulate=False)
            return out
        out = ctx.buffer(out_name, (rows, self.out_features), torch.bfloat16)
        self._library(x, out)
        return out

    def _library(self, x: torch.Tensor, out: torch.Tensor) -> None:
        if self.bias is None:
            torch.matmul(x, self.weight.t(), out=out)
        else:
            torch.addmm(self.bias, x, self.weight.t(), out=out)

    def forward_gated(self, ctx, x: torch.Tensor, out_name: str):
        """For a weight whose rows alternate, in strips of `lib.GATE_STRIP`, between gate rows
        and their up rows: silu(gate) * up as [N, out/2] of the storage type straight from
        the few-rows kernel, or None where that kernel does not apply (float32, many rows, a
        bias, a large matrix whose K the planner would slice); the caller then takes
        `forward` and the activation kernel."""
        rows = x.shape[0]
        if (self.dtype != torch.bfloat16 or self.bias is not None or not lib.skinny_gemm_ok(rows, self.in_features)
                or self.out_features % (2 * lib.GATE_STRIP)
                or (self.weight.numel() * 2 > GATED_UNSLICED_BYTES and
                    lib.skinny_gemm_splits(rows, self.out_features, self.in_features) != 1)):
            return None
        act = ctx.buffer(out_name, (rows, self.out_features // 2), torch.bfloat16)
        packed = self.packed is not None
        lib.gemm_bf16_skinny_gated(x, self.packed if packed else self.weight, self.out_features,
                                   act, packed)
        return act

    def forward_f32(self, ctx, x: torch.Tensor, out_name: str) -> torch.Tensor:
        """Like forward, but one float32 [N, out] tensor (used for the logits)."""
        rows = x.shape[0]
        out = ctx.buffer(out_name, (rows, self.out_features), torch.float32)
        if self.dtype == torch.float32:
            lib.gemm_f32(x, self.weight, out)
            if self.bias is not None:
                lib.bias_rows(self.bias_f32, out, accumulate=True)
            return out
        if self.in_features % 8 == 0:
            # any number of rows, in groups of the few-rows product with its float32 sums: a
            # row's logits are float32 however many rows a step wants (the library's product
            # would round them to bfloat16)
            for start in range(0, rows, SKINNY_ROWS):
                stop = min(rows, start + SKINNY_ROWS)
                count = stop - start
                splits = lib.skinny_gemm_splits(count, self.out_features, self.in_features)
                if splits == 1:
                    self._few_rows(x[start:stop], out[start:stop].unsqueeze(0))
                else:
                    slices = ctx.buffer(out_name + ".slices", (splits, count, self.out_features),
                                        torch.float32)
                    self._few_rows(x[start:stop], slices)
                    lib.sum_slices(slices, out[start:stop])
                    ctx.release(slices)
            if self.bias is not None:
                lib.bias_rows(self.bias_f32, out, accumulate=True)
            return out
        # a width that is no multiple of 8: the library's product, rounded to bfloat16
        low = ctx.buffer(out_name + ".bf16", (rows, self.out_features), torch.bfloat16)
        self._library(x, low)
        out.copy_(low)
        ctx.release(low)
        return out
