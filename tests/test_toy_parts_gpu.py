"""Toy parts defined in this file only — a feed-forward with routing, a position encoding,
a norm and a block arrangement — registered, built and stepped through the engine (whole
sequences and token by token) without a change to the framework's files.  They exist to
show the interfaces; they are nobody's model."""
from dataclasses import dataclass

import pytest
import torch

import plain_qwen3 as plain
from helpers import assert_close_f32
from test_parts_gpu import attention_spec, make_session, mlp_spec, random_params

pytestmark = pytest.mark.gpu
DEV = "cuda"


# ---------------------------------------------------------------------------
# feed-forward with routing: every row goes to the one expert its router prefers
@dataclass(frozen=True)
class RoutedSpec:
    kind: str = "toy_routed"
    n_experts: int = 3
    intermediate_size: int = 24


class RoutedFeedForward:
    """y = gate_e(x) weighted expert e = argmax(router x), each expert a small gated MLP
    (router logits and the softmax weight in float32)."""

    @classmethod
    def parameters(cls, spec, hidden):
        from edge_infer_amd.weights import ParamSpec
        params = {"router.weight": ParamSpec((spec.n_experts, hidden))}
        for e in range(spec.n_experts):
            params[f"experts.{e}.gate_proj.weight"] = ParamSpec((spec.intermediate_size, hidden))
            params[f"experts.{e}.up_proj.weight"] = ParamSpec((spec.intermediate_size, hidden))
            params[f"experts.{e}.down_proj.weight"] = ParamSpec((hidden, spec.intermediate_size))
        return params

    def __init__(self, spec, hidden, params, dtype, device):
        self.spec = spec
        self.params = {k: v.to(device=device, dtype=torch.float32) for k, v in params.items()}

    def forward(self, ctx, x):
        x = x.float()
        logits = x @ self.params["router.weight"].t()
        weight, chosen = torch.softmax(logits, dim=-1).max(dim=-1)
        out = torch.zeros_like(x)
        for e in range(self.spec.n_experts):
            rows = (chosen == e).nonzero().flatten()
            if rows.numel() == 0:
                continue
            h = x[rows]
            g = h @ self.params[f"experts.{e}.gate_proj.weight"].t()
            u = h @ self.params[f"experts.{e}.up_proj.weight"].t()
            y = (torch.nn.functional.silu(g) * u) @ self.params[f"experts.{e}.down_proj.weight"].t()
            out[rows] = y * weight[rows, None]
        return out


def routed_oracle(h, params, prefix, spec):
    logits = plain.linear(h, params[prefix + "router.weight"])
    weight, chosen = torch.softmax(logits, dim=-1).max(dim=-1)
    out = torch.zeros_like(h)
    for r in range(h.shape[0]):
        e = int(chosen[r])
        p = f"{prefix}experts.{e}."
        y = plain.linear(plain.swiglu(plain.linear(h[r:r + 1], params[p + "gate_proj.weight"]),
                                      plain.linear(h[r:r + 1], params[p + "up_proj.weight"])),
                         params[p + "down_proj.weight"])
        out[r] = y[0] * weight[r]
    return out


# ---------------------------------------------------------------------------
# a position encoding: rotation by an angle that grows with the logarithm of the position
@dataclass(frozen=True)
class LogRotarySpec:
    kind: str = "toy_log_rotary"
    dim: int = 16
    max_positions: int = 256
    base: float = 50.0


def log_rotary_angles(spec, positions):
    half = spec.dim // 2
    rate = spec.base ** (-torch.arange(half, dtype=torch.float64) / half)
    return torch.log1p(torch.tensor(positions, dtype=torch.float64))[:, None] * 7.0 * rate[None, :]


class LogRotaryTable:
    """The interface of a position encoding: `.table` float32 [positions, dim], the cosines
    of the dim/2 pairs (i, i + dim/2), then the sines; `.max_positions`."""

    def __init__(self, spec, device):
        angle = log_rotary_angles(spec, list(range(spec.max_positions)))
        self.table = torch.cat([torch.cos(angle), torch.sin(angle)], dim=1).float().to(device)
        self.max_positions = spec.max_positions


def rotate(x, angle):
    """x [S, heads, d] rotated pairwise (i, i + d/2) by angle [S, d/2] (float64)."""
    half = x.shape[-1] // 2
    cos, sin = torch.cos(angle)[:, None, :], torch.sin(angle)[:, None, :]
    a, b = x[..., :half], x[..., half:]
    return torch.cat([a * cos - b * sin, a * sin + b * cos], dim=-1)


# ---------------------------------------------------------------------------
# a norm: mean-centred, scaled to unit variance, weight and bias
@dataclass(frozen=True)
class CentredNormSpec:
    kind: str = "toy_centred_norm"
    eps: float = 1e-5


class CentredNorm:
    @classmethod
    def parameters(cls, spec, width):
        from edge_infer_amd.weights import ParamSpec
        return {"weight": ParamSpec((width,), init="norm"), "bias": ParamSpec((width,))}

    def __init__(self, spec, width, params, dtype, device):
        self.eps = spec.eps
        self.width = width
        self.weight = params["weight"].to(device=device, dtype=torch.float32)
        self.bias = params["bias"].to(device=device, dtype=torch.float32)

    def add_norm(self, ctx, residual, delta, out_name, rows=None, write_residual=True):
        """residual += delta (summed over its slices if it has any); the normed rows."""
        total = residual
        if delta is not None:
            d = delta.float()
            total = residual + (d.sum(0) if d.dim() == 3 else d)
            if write_residual:
                residual.copy_(total)
        picked = total if rows is None else total[rows.long()]
        centred = picked - picked.mean(-1, keepdim=True)
        normed = centred * torch.rsqrt(centred.pow(2).mean(-1, keepdim=True) + self.eps)
        out = ctx.buffer(out_name, (picked.shape[0], self.width))
        out.copy_(normed * self.weight + self.bias)
        return out


def centred_norm_oracle(x, weight, bias, eps):
    centred = x - x.mean(-1, keepdim=True)
    return centred / torch.sqrt(centred.pow(2).mean(-1, keepdim=True) + eps) * weight.double() + bias.double()


# ---------------------------------------------------------------------------
# a block arrangement: mixer and feed-forward both read the same normed input
class ParallelBlock:
    """x += mixer(norm(x)) + feed_forward(norm(x)), one norm per layer."""

    @classmethod
    def parameters(cls, layer_spec, hidden):
        from edge_infer_amd.parts import lookup
        params = {}
        for prefix, family, spec in (("norm", "norm", layer_spec.norm),
                                     ("mixer", "mixer", layer_spec.mixer),
                                     ("ffn", "feed_forward", layer_spec.feed_forward)):
            for name, param in lookup(family, spec.kind).parameters(spec, hidden).items():
                params[f"{prefix}.{name}"] = param
        return params

    @classmethod
    def mixer_spec(cls, layer_spec):
        return layer_spec.mixer

    def __init__(self, layer_spec, hidden, params, dtype, device, positions):
        from edge_infer_amd.parts import lookup

        def sub(prefix):
            return {k[len(prefix) + 1:]: v for k, v in params.items() if k.startswith(prefix + ".")}
        self.norm = lookup("norm", layer_spec.norm.kind)(layer_spec.norm, hidden, sub("norm"),
                                                         dtype, device)
        self.mixer = lookup("mixer", layer_spec.mixer.kind)(layer_spec.mixer, hidden, sub("mixer"),
                                                            dtype, device, positions=positions)
        self.ffn = lookup("feed_forward", layer_spec.feed_forward.kind)(
            layer_spec.feed_forward, hidden, sub("ffn"), dtype, device)

    def forward(self, ctx, residual, pending, entry):
        h = self.norm.add_norm(ctx, residual, pending, "block.h")
        a = self.mixer.forward(ctx, h, entry)
        f = self.ffn.forward(ctx, h)
        a = a.float().sum(0) if a.dim() == 3 else a.float()
        f = f.float().sum(0) if f.dim() == 3 else f.float()
        return a + f                         # left pending: the next norm adds it


# ---------------------------------------------------------------------------
def test_toy_feed_forward_position_norm_and_block_through_the_engine():
    from edge_infer_amd.config.specs import LayerSpec, ModelSpec, NormSpec, ScheduleEntry
    from edge_infer_amd.parts import (register_block, register_feed_forward, register_norm,
                                      register_position, unregister)
    hidden, vocab = 40, 61
    register_feed_forward("toy_routed", RoutedFeedForward)
    register_position("toy_log_rotary", LogRotaryTable)
    register_norm("toy_centred_norm", CentredNorm)
    register_block("toy_parallel", ParallelBlock)
    try:
        rms, centred = NormSpec(eps=1e-5), CentredNormSpec()
        log_rotary = LogRotarySpec(dim=16, max_positions=256)
        routed = RoutedSpec(n_experts=3, intermediate_size=24)
        layers = (
            # the framework's attention with the toy position encoding and the toy routed FFN
            LayerSpec("prenorm", rms, attention_spec(position=log_rotary), routed),
            # the toy norm and the toy arrangement around the framework's attention and MLP
            LayerSpec("toy_parallel", centred, attention_spec(n_heads=4, n_kv_heads=4), mlp_spec(48)),
        )
        spec = ModelSpec(architecture="ToyPartsForCausalLM", vocab_size=vocab, hidden_size=hidden,
                         layers=layers, schedule=(ScheduleEntry(0, 0), ScheduleEntry(1, 1)),
                         final_norm=rms, tie_word_embeddings=False, max_position_embeddings=256,
                         bos_token_id=0, eos_token_id=1)
        params = random_params(spec, 21)
        params = {k: (v * 4 if "router" in k else v) for k, v in params.items()}
        model, session = make_session(spec, params, max_tokens=512, max_seqs=3)

        def attention(layer, h, mixer, angle):
            S = h.shape[0]
            p = f"layers.{layer}.mixer."
            q = plain.linear(h, params[p + "q_proj.weight"]).reshape(S, mixer.n_heads, mixer.head_dim)
            k = plain.linear(h, params[p + "k_proj.weight"]).reshape(S, mixer.n_kv_heads, mixer.head_dim)
            v = plain.linear(h, params[p + "v_proj.weight"]).reshape(S, mixer.n_kv_heads, mixer.head_dim)
            q = plain.rms_norm(q, params[p + "q_norm.weight"], mixer.qk_norm_eps)
            k = plain.rms_norm(k, params[p + "k_norm.weight"], mixer.qk_norm_eps)
            if angle is None:
                q = plain.rope(q, list(range(S)), mixer.position.theta)
                k = plain.rope(k, list(range(S)), mixer.position.theta)
            else:
                q, k = rotate(q, angle), rotate(k, angle)
            return plain.linear(plain.attention(q, k, v).reshape(S, -1), params[p + "o_proj.weight"])

        def oracle(ids):
            S = len(ids)
            x = plain.embedding(ids, params["embed.weight"])
            h = plain.rms_norm(x, params["layers.0.norm1.weight"], 1e-5)
            x = x + attention(0, h, layers[0].mixer, log_rotary_angles(log_rotary, list(range(S))))
            h = plain.rms_norm(x, params["layers.0.norm2.weight"], 1e-5)
            x = x + routed_oracle(h, {k: v.double() for k, v in params.items()}, "layers.0.ffn.", routed)
            h = centred_norm_oracle(x, params["layers.1.norm.weight"], params["layers.1.norm.bias"],
                                    centred.eps)
            f = plain.linear(plain.swiglu(plain.linear(h, params["layers.1.ffn.gate_proj.weight"]),
                                          plain.linear(h, params["layers.1.ffn.up_proj.weight"])),
                             params["layers.1.ffn.down_proj.weight"])
            x = x + attention(1, h, layers[1].mixer, None) + f
            return plain.linear(plain.rms_norm(x, params["final_norm.weight"], 1e-5),
                                params["head.weight"])

        g = torch.Generator().manual_seed(4)
        a = torch.randint(0, vocab, (70,), generator=g).tolist()
        b = torch.randint(0, vocab, (23,), generator=g).tolist()
        ref_a, ref_b = oracle(a), oracle(b)
        # more than one expert is in use, or the routing shows nothing
        h0 = plain.rms_norm(plain.embedding(a, params["embed.weight"]), params["layers.0.norm1.weight"], 1e-5)
        assert len(set(plain.linear(h0, params["layers.0.ffn.router.weight"]).argmax(-1).tolist())) > 1

        sa, sb = session.begin(), session.begin()
        logits = session.step([(sa, a, list(range(70))), (sb, b, list(range(23)))])
        assert_close_f32(logits[:70], ref_a, "toy parts whole a")
        assert_close_f32(logits[70:], ref_b, "toy parts whole b")
        session.end(sa)
        session.end(sb)
        # a prefix, then token by token, in slots that are used again
        sb, sa = session.begin(), session.begin()
        first = session.step([(sa, a[:50], [49]), (sb, b[:3], [2])])
        got_a, got_b = [first[0]], [first[1]]
        for t in range(20):
            out = session.step([(sa, [a[50 + t]], [0]), (sb, [b[3 + t]], [0])])
            got_a.append(out[0])
            got_b.append(out[1])
        assert_close_f32(torch.stack(got_a), ref_a[49:], "toy parts decode a")
        assert_close_f32(torch.stack(got_b), ref_b[2:23], "toy parts decode b")
    finally:
        unregister("feed_forward", "toy_routed")
        unregister("position", "toy_log_rotary")
        unregister("norm", "toy_centred_norm")
        unregister("block", "toy_parallel")
