"""The decoder model: embedding, the layers in schedule order, final norm, head.

`DecoderModel` is built from a `ModelSpec` and a dictionary of parameters; it owns
immutable weights on the device and nothing that changes between steps (sessions
own caches and workspaces).  Its `forward` is the one step function: it runs the
rows of a `StepContext` and returns float32 logits at the wanted rows.

Order of operations: runtime/include/execution/decoder.hpp:109-171 and
runtime/src/qwen3.cpp:293-299 of the reference (embedding, blocks, final norm,
head); the head is applied to the wanted rows only.

The skeleton around the layers is four methods, each of which an architecture may
replace in a subclass that it registers as its `model_factory`, keeping the rest:

  embed_rows(ctx) -> residual                 float32 [rows, hidden] in the buffer "residual"
  run_layers(ctx, residual) -> pending        the layers in schedule order; the last delta,
                                              not yet added to the residual
  final_hidden(ctx, residual, pending) -> h   [wanted rows, hidden] in the storage type
  logits(ctx, h) -> float32 [wanted rows, vocab]

(a scaled embedding overrides `embed`, a cap on the logits `logits`, a model without a
final norm `final_hidden`).  A subclass whose methods launch anything that a HIP graph
cannot hold says so with `seams_capture_safe = False`; decode then runs eagerly.
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


def _round_up_fine(count: int) -> int:
    """The next multiple of an eighth of the power of two at or below `count`: at most an
    eighth above it."""
    if count <= 8:
        return count
    step = 1 << (count.bit_length() - 4)
    return (count + step - 1) // step * step


def _round_up_coarse(count: int) -> int:
    return 1 << max(0, (count - 1).bit_length())


FEW_ROWS = 256


def workspace_class(ctx):
    """(signature, scale) under which a step's buffers are planned.  Decode steps and steps
    of few rows are planned for their exact shape (the few-rows product slices K differently
    for every row count).  Prompt steps of more rows share a plan with every step of about
    their size: rows rounded up by at most an eighth, sequences and wanted rows to a power of
    two (wanted rows that are all rows follow the rows); the recorded sizes are scaled to the
    largest step of the class, which is safe because every buffer of such a step is at most
    linear in rows, sequences and wanted rows."""
    rows, seqs, want = ctx.n_rows, ctx.n_seqs, ctx.meta.n_want
    bound = ctx.context_bound if ctx.fixed_shape else None
    if ctx.decode or rows <= FEW_ROWS:
        return (rows, seqs, want, ctx.decode, bound), 1.0
    rows_up, seqs_up = _round_up_fine(rows), _round_up_coarse(seqs)
    if want == rows:
        want_up, want_key = rows_up, "all"
    elif want == 0:
        want_up = want_key = 0
    else:
        want_up = want_key = _round_up_coarse(want)
    scale = max(rows_up / rows, seqs_up / seqs, want_up / max(1, want))
    return (rows_up, seqs_up, want_key, False, bound), scale


def members_of(block):
    """The parts a block holds: what its `members()` names, or else every attribute of it
    that is a part (has `forward` or `add_norm`).  The model asks them, not the block, what
    they plan for a step and whether they can be captured, so a block arrangement is only
    an order of calls."""
    if hasattr(block, "members"):
        return tuple(block.members())
    return tuple(part for part in vars(block).values()
                 if hasattr(part, "forward") or hasattr(part, "add_norm"))


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
        lib.prepare(self.kernel_libraries(spec, self.dtype))
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

    @staticmethod
    def kernel_libraries(spec: ModelSpec, dtype):
        """The kernel libraries a model of `spec` will run, as its parts' classes tell
        (`kernel_libraries(spec, dtype)`, optional): they are compiled side by side before the
        model is made, where they are not built yet, instead of one after the other at their
        first use."""
        names = ["rowwise", *Linear.kernel_libraries(dtype)]        # embedding, norms, head
        for layer in spec.layers:
            ask = getattr(lookup("block", layer.block), "kernel_libraries", None)
            if ask is not None:
                names.extend(ask(layer, dtype))
        return tuple(dict.fromkeys(names))

    def position_table(self, position_spec):
        """One shared encoding object per distinct position spec."""
        table = self._positions.get(position_spec)
        if table is None:
            table = lookup("position", position_spec.kind)(position_spec, self.device)
            self._positions[position_spec] = table
        return table

    def max_positions(self) -> int:
        limit = self.spec.max_position_embeddings
        for table in self._positions.values():
            if table.max_positions is not None:
                limit = min(limit, table.max_positions)
        return limit

    def _planners(self):
        """The parts that plan metadata sections of their own, each kind once: parts that
        would plan the same sections say so with an equal `plan_key` (36 attention layers of
        one shape plan one work list, not 36)."""
        found = getattr(self, "_planner_list", None)
        if found is None:
            found, seen = [], set()
            for layer in self.layers:
                for part in (layer, *members_of(layer)):
                    if not hasattr(part, "plan_step"):
                        continue
                    key = getattr(part, "plan_key", None)
                    if key is not None:
                        if key in seen:
                            continue
                        seen.add(key)
                    found.append(part)
            self._planner_list = found
        return found

    def plan_step(self, plan) -> None:
        """Let the parts add the metadata sections they plan for themselves (work items of
        their kernels and the like) to the step plan; the engine only carries them."""
        for part in self._planners():
            plan.add_sections(part.plan_step(plan))

    seams_capture_safe = True     # embed / final_hidden / logits launch only capturable work

    def capture_safe(self) -> bool:
        """Whether a decode step may be captured in a HIP graph: the final norm, the head,
        every block and every part of a block must say so with `capture_safe` (it launches
        nothing but capturable kernels and allocates nothing per step; a part that does not
        say so is taken to be unsafe), and so must the model's own methods around them."""
        if not self.seams_capture_safe:
            return False
        parts = [self.final_norm, self.head]
        for layer in self.layers:
            parts += [layer, *members_of(layer)]
        return all(bool(getattr(part, "capture_safe", False)) for part in parts)

    def capture_rows(self) -> int:
        """Most rows of a step for which `capture_safe` holds: the least any part allows."""
        rows = self.head.capture_rows
        for layer in self.layers:
            for part in (layer, *members_of(layer)):
                rows = min(rows, getattr(part, "capture_rows", 1 << 30))
        return rows

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
        and, for a captured step, the context bound that fixes the parts' launch shapes."""
        workspace = ctx.workspace
        workspace.start(*workspace_class(ctx))
        try:
            logits = self._forward(ctx)
        except BaseException:
            workspace.abort()
            raise
        workspace.finish()
        return logits

    def _forward(self, ctx) -> torch.Tensor:
        residual = self.embed_rows(ctx)
        pending = self.run_layers(ctx, residual)
        if ctx.meta.n_want == 0:
            return torch.empty((0, self.spec.vocab_size), dtype=torch.float32,
                               device=self.device)
        hidden = self.final_hidden(ctx, residual, pending)
        ctx.release(pending)
        return self.logits(ctx, hidden)

    # -- the skeleton: what a subclass may replace -------------------------------
    def embed_rows(self, ctx) -> torch.Tensor:
        """The rows of the embedding table that the step's tokens name, as the float32
        residual stream [rows, hidden]."""
        residual = ctx.buffer("residual", (ctx.n_rows, self.spec.hidden_size), torch.float32)
        lib.embed_gather(ctx.meta.tokens, self.embed, residual)
        return residual

    def run_layers(self, ctx, residual):
        """The layers in the order of the schedule.  Returns the last delta, which is not
        added to the residual yet (the norm that follows adds it while it reads the row)."""
        pending = None
        for entry in self.spec.schedule:
            pending = self.layers[entry.layer].forward(ctx, residual, pending, entry)
        return pending

    def final_hidden(self, ctx, residual, pending) -> torch.Tensor:
        """The normalised rows that the head reads: only the wanted ones."""
        return self.final_norm.add_norm(ctx, residual, pending, "final.h",
                                        rows=ctx.meta.want_rows, write_residual=False)

    def logits(self, ctx, hidden) -> torch.Tensor:
        """float32 [wanted rows, vocab] in the buffer "logits"."""
        return self.head.forward_f32(ctx, hidden, "logits")
