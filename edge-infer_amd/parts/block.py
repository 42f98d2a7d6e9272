"""Arrangements of norm, mixer and feed-forward in one layer."""
from __future__ import annotations

from .registry import lookup


class PreNormBlock:
    """x += mixer(norm1(x)); x += feed_forward(norm2(x)).
    runtime/include/execution/decoder.hpp:119-168 of the reference.  The second
    addition is left pending: the next block's first norm (or the model's final
    norm) performs it while reading the row."""

    parts = ("norm1", "mixer", "norm2", "ffn")
    capture_safe = True      # nothing of its own besides its parts' kernels

    def members(self):
        """The parts this block is made of, in the order in which they run."""
        return (self.norm1, self.mixer, self.norm2, self.ffn)

    @classmethod
    def parameters(cls, layer_spec, hidden):
        norm_cls = lookup("norm", layer_spec.norm.kind)
        mixer_cls = lookup("mixer", layer_spec.mixer.kind)
        ffn_cls = lookup("feed_forward", layer_spec.feed_forward.kind)
        params = {}
        for prefix, owner, spec in (("norm1", norm_cls, layer_spec.norm),
                                    ("mixer", mixer_cls, layer_spec.mixer),
                                    ("norm2", norm_cls, layer_spec.norm),
                                    ("ffn", ffn_cls, layer_spec.feed_forward)):
            for name, param in owner.parameters(spec, hidden).items():
                params[f"{prefix}.{name}"] = param
        return params

    @classmethod
    def mixer_spec(cls, layer_spec):
        return layer_spec.mixer

    @classmethod
    def kernel_libraries(cls, layer_spec, dtype):
        """The kernel libraries its parts say they run (a part without the method says none)."""
        names = []
        for category, spec in (("norm", layer_spec.norm), ("mixer", layer_spec.mixer),
                               ("feed_forward", layer_spec.feed_forward)):
            ask = getattr(lookup(category, spec.kind), "kernel_libraries", None)
            if ask is not None:
                names.extend(ask(spec, dtype))
        return tuple(names)

    def __init__(self, layer_spec, hidden, params, dtype, device, positions):
        def sub(prefix):
            return {name[len(prefix) + 1:]: tensor for name, tensor in params.items()
                    if name.startswith(prefix + ".")}
        norm_cls = lookup("norm", layer_spec.norm.kind)
        mixer_cls = lookup("mixer", layer_spec.mixer.kind)
        ffn_cls = lookup("feed_forward", layer_spec.feed_forward.kind)
        self.norm1 = norm_cls(layer_spec.norm, hidden, sub("norm1"), dtype, device)
        self.mixer = mixer_cls(layer_spec.mixer, hidden, sub("mixer"), dtype, device,
                               positions=positions)
        self.norm2 = norm_cls(layer_spec.norm, hidden, sub("norm2"), dtype, device)
        self.ffn = ffn_cls(layer_spec.feed_forward, hidden, sub("ffn"), dtype, device)

    def forward(self, ctx, residual, pending, entry):
        h = self.norm1.add_norm(ctx, residual, pending, "block.h")
        ctx.release(pending)             # added into the residual: its storage is free
        a = self.mixer.forward(ctx, h, entry)
        ctx.release(h)
        h2 = self.norm2.add_norm(ctx, residual, a, "block.h")
        ctx.release(a)
        out = self.ffn.forward(ctx, h2)
        ctx.release(h2)
        return out
