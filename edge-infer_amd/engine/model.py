"""The decoder model: embedding, the layers in schedule order, final norm, head.

`DecoderModel` is built from a `ModelSpec` and a dictionary of parameters; it owns
immutable weights on the device and nothing that changes between steps (sessions
own caches and workspaces).  Its `forward` is the one step function: it runs the
rows of a `StepContext` and returns float32 logits at the wanted rows.

Order of operations: runtime/include/execution/decoder.hpp:109-171 and
runtime/src/qwen3.cpp:293-299 of the reference (embedding, blocks, final norm,
head); the head is applied to the wanted rows only.
"""
from __future__ import annotations

from typing import Callable, Dict, Mapping, Tuple

import torch

from ..config.specs import ModelSpec
from ..csrc import lib
from ..parts.linear import Linear
from ..parts.registry import lookup
from ..weights.loader import ParamSpec

DTYPES = {"float32": torch.float32, "fp32": torch.float32, "bfloat16": torch.bfloat16,
          "bf16": torch.bfloat16, torch.float32: torch.float32, torch.bfloat16: torch.bfloat16}


def resolve_dtype(dtype):
    try:
        return DTYPES[dtype]
    except KeyError:
        raise ValueError(f"dtype must be 'bfloat16' or 'float32', got {dtype!r}") from None


def model_parameters(spec: ModelSpec) -> Dict[str, ParamSpec]:
    """Every parameter of the model by its path."""
    params = {"embed.weight": ParamSpec((spec.vocab_size, spec.hidden_size))}
    for index, layer in enumerate(spec.layers):
        block_cls = lookup("block", layer.block)
        for name, param in block_cls.parameters(layer, spec.hidden_size).items():
            params[f"layers.{index}.{name}"] = param
    final_cls = lookup("norm", spec.final_norm.kind)
    for name, param in final_cls.parameters(spec.final_norm, spec.hidden_size).items():
        params[f"final_norm.{name}"] = param
    params["head.weight"] = ParamSpec((spec.vocab_size, spec.hidden_size))
    params["head.bias"] = ParamSpec((spec.vocab_size,), optional=True)
    return params


def expected_parameters(spec: ModelSpec, checkpoint_name: Callable[[str], str]
                        ) -> Dict[str, Tuple[str, ParamSpec]]:
    """parameter path -> (checkpoint tensor name, spec)."""
    return {path: (checkpoint_name(path), param)
            for path, param in model_parameters(spec).items()}


class DecoderModel:
    def __init__(self, spec: ModelSpec, params: Mapping[str, torch.Tensor], dtype, device):
        spec.validate()
        self.spec = spec
        self.dtype = resolve_dtype(dtype)
        self.device = torch.device(device)
        wanted = model_parameters(spec)
        missing = [p for p, param in wanted.items() if p not in params and not param.optional
                   and not (p == "head.weight" and spec.tie_word_embeddings)]
        if missing:
            raise KeyError(f"model parameters missing: {missing}")
        self._positions = {}
        self.embed = params["embed.weight"].to(device=self.device, dtype=self.dtype).contiguous()
        self.layers = []
        for index, layer in enumerate(spec.layers):
            prefix = f"layers.{index}."
            own = {name[len(prefix):]: tensor for name, tensor in params.items()
                   if name.startswith(prefix)}
            block_cls = lookup("block", layer.block)
            self.layers.append(block_cls(layer, spec.hidden_size, own, self.dtype, self.device,
                                         positions=self.position_table))
        final_cls = lookup("norm", spec.final_norm.kind)
        self.final_norm = final_cls(spec.final_norm, spec.hidden_size,
                                    {"weight": params["final_norm.weight"]}, self.dtype,
                                    self.device)
        if "head.weight" in params and params["head.weight"] is not params["embed.weight"]:
            self.head = Linear(params["head.weight"], self.dtype, self.device,
                               bias=params.get("head.bias"))
        else:  # tied: the head is the embedding table itself (no copy: same type and device)
            self.head = Linear(self.embed, self.dtype, self.device, bias=params.get("head.bias"))

    def position_table(self, position_spec):
        """One shared encoding object per distinct position spec."""
        table = self._positions.get(position_spec)
        if table is None:
            table = lookup("position", position_spec.kind)(position_spec, self.device)
            self._positions[position_spec] = table
        return table

    def attention_item_sizes(self):
        sizes = set()
        for layer in self.layers:
            mixer = getattr(layer, "mixer", None)
            if mixer is not None and hasattr(mixer, "positions_per_item"):
                sizes.add(mixer.positions_per_item())
        return tuple(sorted(sizes))

    def max_positions(self) -> int:
        limit = self.spec.max_position_embeddings
        for table in self._positions.values():
            if table.max_positions is not None:
                limit = min(limit, table.max_positions)
        return limit

    def capture_safe(self) -> bool:
        """Whether a decode step may be captured in a HIP graph: every block and every
        part that a block holds (norms, mixer, feed-forward) must say so with
        `capture_safe = True` (it launches nothing but capturable kernels and allocates
        nothing per step; a part that does not say so is taken to be unsafe), and every
        linear layer must take the hand-written kernel for few rows (library products may
        record memset nodes, which are not replayed reliably)."""
        def linears(obj, depth=0):
            if isinstance(obj, Linear):
                yield obj
            elif depth < 3 and hasattr(obj, "__dict__"):
                for value in vars(obj).values():
                    yield from linears(value, depth + 1)
        if not getattr(self.final_norm, "capture_safe", False):
            return False
        for layer in self.layers:
            if not getattr(layer, "capture_safe", False):
                return False
            for part in vars(layer).values():
                if hasattr(part, "forward") or hasattr(part, "add_norm"):
                    if not getattr(part, "capture_safe", False):
                        return False
            for linear in linears(layer):
                if linear.dtype == torch.bfloat16 and linear.in_features % 8:
                    return False
        if self.head.dtype == torch.bfloat16 and self.head.in_features % 8:
            return False
        return True

    def weight_bytes(self) -> int:
        seen, total = set(), 0

        def visit(obj):
            nonlocal total
            if isinstance(obj, torch.Tensor):
                if obj.data_ptr() not in seen:
                    seen.add(obj.data_ptr())
                    total += obj.numel() * obj.element_size()
            elif hasattr(obj, "__dict__"):
                for value in vars(obj).values():
                    visit(value)
        visit(self.embed)
        for layer in self.layers:
            visit(layer)
        visit(self.final_norm)
        visit(self.head)
        return total

    # ------------------------------------------------------------------
    def forward(self, ctx) -> torch.Tensor:
        """Run the rows of `ctx`; float32 logits [wanted rows, vocab].  The step's buffers
        are planned by the workspace per shape of step: rows, sequences, wanted rows, kind,
        and the context bound that fixes the launch shape of decode attention."""
        workspace = ctx.workspace
        workspace.start((ctx.n_rows, ctx.n_seqs, ctx.meta.n_want, ctx.decode,
                         getattr(ctx, "_fixed_context", None)))
        try:
            logits = self._forward(ctx)
        except BaseException:
            workspace.abort()
            raise
        workspace.finish()
        return logits

    def _forward(self, ctx) -> torch.Tensor:
        spec = self.spec
        meta = ctx.meta
        residual = ctx.buffer("residual", (ctx.n_rows, spec.hidden_size), torch.float32)
        lib.embed_gather(meta.tokens, self.embed, residual)
        pending = None
        for entry in spec.schedule:
            pending = self.layers[entry.layer].forward(ctx, residual, pending, entry)
        if meta.n_want == 0:
            return torch.empty((0, spec.vocab_size), dtype=torch.float32, device=self.device)
        hidden = self.final_norm.add_norm(ctx, residual, pending, "final.h", rows=meta.want_rows,
                                          write_residual=False)
        ctx.release(pending)
        return self.head.forward_f32(ctx, hidden, "logits")
