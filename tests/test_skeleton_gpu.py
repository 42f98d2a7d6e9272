"""What another architecture may differ in without a change to the framework's files, shown
with toy parts that this file defines: a model class of its own around the layers (an
embedding that is scaled, logits that are capped), registered as the architecture's model
and built through every path (`random_model`, a model folder); a rotation that covers only
part of every head; a cache whose values are narrower than its keys.  They are nobody's
model."""
import json
import math
from dataclasses import dataclass

import pytest
import torch

import plain_qwen3 as plain
from helpers import assert_close, assert_close_f32, random_ids
from test_parts_gpu import attention_spec, make_session, mlp_spec, one_layer_spec, random_params

pytestmark = pytest.mark.gpu
DEV = "cuda"


# ---------------------------------------------------------------------------
# an architecture whose skeleton differs: scaled embedding, capped logits
@dataclass(frozen=True)
class ToySkeletonConfig:
    vocab_size: int = 211
    hidden_size: int = 48
    layers: int = 2
    heads: int = 3
    head_dim: int = 16
    intermediate_size: int = 80
    cap: float = 1.5
    max_positions: int = 256

    architecture = "ToySkeletonForCausalLM"

    @classmethod
    def from_dict(cls, raw):
        return cls(**{key: raw[key] for key in cls.__dataclass_fields__ if key in raw})

    def to_dict(self):
        return dict(architectures=[self.architecture],
                    **{key: getattr(self, key) for key in self.__dataclass_fields__})

    def model_spec(self):
        from edge_infer_amd.config.specs import (AttentionSpec, GatedMLPSpec, LayerSpec, ModelSpec,
                                                 NormSpec, PositionSpec, default_schedule)
        norm = NormSpec(eps=1e-5)
        mixer = AttentionSpec(n_heads=self.heads, n_kv_heads=1, head_dim=self.head_dim,
                              qk_norm=True, qk_norm_eps=1e-5,
                              position=PositionSpec(kind="rope", theta=1e4, dim=self.head_dim,
                                                    max_positions=self.max_positions))
        layer = LayerSpec("prenorm", norm, mixer, GatedMLPSpec(intermediate_size=self.intermediate_size))
        return ModelSpec(architecture=self.architecture, vocab_size=self.vocab_size,
                         hidden_size=self.hidden_size, layers=(layer,) * self.layers,
                         schedule=default_schedule(self.layers), final_norm=norm,
                         tie_word_embeddings=True, max_position_embeddings=self.max_positions,
                         bos_token_id=0, eos_token_id=1)

    @staticmethod
    def checkpoint_name(parameter):
        return "toy." + parameter


def toy_skeleton_model_class():
    from edge_infer_amd.engine.model import DecoderModel

    class ToySkeletonModel(DecoderModel):
        """embedding * sqrt(hidden) in front, cap * tanh(logits / cap) behind: two of the four
        methods of the skeleton replaced, the layers and the final norm kept."""

        def embed_rows(self, ctx):
            residual = super().embed_rows(ctx)
            return residual.mul_(math.sqrt(self.spec.hidden_size))

        def logits(self, ctx, hidden):
            cap = self.config.cap if hasattr(self, "config") else ToySkeletonConfig.cap
            logits = super().logits(ctx, hidden)
            return logits.div_(cap).tanh_().mul_(cap)

    return ToySkeletonModel


def toy_skeleton_oracle(cfg, weights, ids, rope=plain.rope, scaled_and_capped=True):
    """The same model from the plain parts, float64."""
    S = len(ids)
    name = cfg.checkpoint_name
    x = plain.embedding(ids, weights[name("embed.weight")])
    if scaled_and_capped:
        x = x * math.sqrt(cfg.hidden_size)
    for layer in range(cfg.layers):
        p = f"layers.{layer}."
        h = plain.rms_norm(x, weights[name(p + "norm1.weight")], 1e-5)
        q = plain.linear(h, weights[name(p + "mixer.q_proj.weight")]).reshape(S, cfg.heads, cfg.head_dim)
        k = plain.linear(h, weights[name(p + "mixer.k_proj.weight")]).reshape(S, 1, cfg.head_dim)
        v = plain.linear(h, weights[name(p + "mixer.v_proj.weight")]).reshape(S, 1, cfg.head_dim)
        q = rope(plain.rms_norm(q, weights[name(p + "mixer.q_norm.weight")], 1e-5), range(S), 1e4)
        k = rope(plain.rms_norm(k, weights[name(p + "mixer.k_norm.weight")], 1e-5), range(S), 1e4)
        x = x + plain.linear(plain.attention(q, k, v).reshape(S, -1),
                             weights[name(p + "mixer.o_proj.weight")])
        h = plain.rms_norm(x, weights[name(p + "norm2.weight")], 1e-5)
        x = x + plain.linear(plain.swiglu(plain.linear(h, weights[name(p + "ffn.gate_proj.weight")]),
                                          plain.linear(h, weights[name(p + "ffn.up_proj.weight")])),
                             weights[name(p + "ffn.down_proj.weight")])
    logits = plain.linear(plain.rms_norm(x, weights[name("final_norm.weight")], 1e-5),
                          weights[name("embed.weight")])
    return cfg.cap * torch.tanh(logits / cfg.cap) if scaled_and_capped else logits


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_an_architecture_with_a_model_class_of_its_own(tmp_path, dtype):
    """Registered with a model factory, the architecture gets its class from a folder, from
    `random_model` and from `api.Model`, steps whole and token by token (from graphs: the
    replaced methods only launch work a graph can hold), and matches its plain form."""
    import edge_infer_amd as ei
    from edge_infer_amd.config import register_architecture, unregister_architecture
    model_class = toy_skeleton_model_class()
    register_architecture("ToySkeletonForCausalLM", ToySkeletonConfig, model_factory=model_class,
                          model_types=("toy_skeleton",))
    try:
        cfg = ToySkeletonConfig()
        folder = ei.write_model_folder(tmp_path / "toy", cfg, seed=8)
        # embedding rows large enough for the cap to bend the logits
        from safetensors.torch import load_file, save_file
        tensors = load_file(str(folder / "model.safetensors"))
        tensors = {k: (v.float() * 6).to(torch.bfloat16) if k == "toy.embed.weight" else v
                   for k, v in tensors.items()}
        save_file(tensors, str(folder / "model.safetensors"))
        assert json.loads((folder / "config.json").read_text())["cap"] == 1.5
        model = ei.load_model(folder, dtype=dtype)
        assert type(model) is model_class and model.config == cfg
        assert type(ei.random_model(cfg, seed=8, dtype=dtype)) is model_class
        weights = {k: v.double() for k, v in tensors.items()}
        ids = random_ids(cfg.vocab_size, 60, 5)
        want = toy_skeleton_oracle(cfg, weights, ids)
        assert want.abs().max() > 0.8 * cfg.cap, "the cap was meant to matter"
        session = ei.Session(model, max_tokens=128, max_seqs=2)
        assert session.graphs
        slot = session.begin()
        rows = [session.step([(slot, ids[:40], list(range(40)))])]
        rows += [session.step([(slot, [token], [0])]) for token in ids[40:]]
        assert session.graph_replays > 0
        assert_close(dtype, torch.cat(rows), want, f"{dtype} toy skeleton")
    finally:
        unregister_architecture("ToySkeletonForCausalLM")
    with pytest.raises(KeyError):
        ei.load_model(folder, dtype=dtype)


# ---------------------------------------------------------------------------
# an architecture whose checkpoints rotate neighbouring elements (2j, 2j + 1) instead of the
# halves (j, j + d/2): no kernel and no position part of its own.  A query and a key give the
# same score when both are permuted alike, so the architecture's model factory reorders the
# rows of its q and k projections (and the per-head norm weights) once, when the model is built.
@dataclass(frozen=True)
class ToyNeighbourPairsConfig(ToySkeletonConfig):
    architecture = "ToyNeighbourPairsForCausalLM"


def neighbour_pairs_factory(spec, params, dtype, device):
    from edge_infer_amd.engine.model import DecoderModel
    d = spec.layers[0].mixer.head_dim
    order = torch.cat([torch.arange(0, d, 2), torch.arange(1, d, 2)])    # evens, then odds

    def per_head(rows):
        return rows.reshape(-1, d, *rows.shape[1:])[:, order].reshape(rows.shape)

    ordered = dict(params)
    for name, tensor in params.items():
        if name.endswith(("mixer.q_proj.weight", "mixer.k_proj.weight")):
            ordered[name] = per_head(tensor)
        elif name.endswith(("mixer.q_norm.weight", "mixer.k_norm.weight")):
            ordered[name] = tensor[order]
    return DecoderModel(spec, ordered, dtype, device)


def neighbour_pair_rope(x, positions, theta):
    """x [S, heads, d]: elements (2j, 2j + 1) of a head as one complex number, multiplied by
    e^(i p theta^(-2j/d)) at position p."""
    S, heads, d = x.shape
    p = torch.tensor(list(positions), dtype=torch.float64)
    frequency = theta ** (-torch.arange(0, d, 2, dtype=torch.float64) / d)
    turn = torch.polar(torch.ones(S, d // 2, dtype=torch.float64), p[:, None] * frequency[None])
    z = torch.view_as_complex(x.double().reshape(S, heads, d // 2, 2).contiguous()) * turn[:, None]
    return torch.view_as_real(z).reshape(S, heads, d)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_checkpoint_that_rotates_neighbouring_elements(tmp_path, dtype):
    import edge_infer_amd as ei
    from edge_infer_amd.config import register_architecture, unregister_architecture
    from safetensors.torch import load_file
    register_architecture(ToyNeighbourPairsConfig.architecture, ToyNeighbourPairsConfig,
                          model_factory=neighbour_pairs_factory)
    try:
        cfg = ToyNeighbourPairsConfig(max_positions=512)
        folder = ei.write_model_folder(tmp_path / "pairs", cfg, seed=12)
        weights = {k: v.double() for k, v in load_file(str(folder / "model.safetensors")).items()}
        ids = random_ids(cfg.vocab_size, 300, 6)
        want = toy_skeleton_oracle(cfg, weights, ids, rope=neighbour_pair_rope,
                                   scaled_and_capped=False)
        halves = toy_skeleton_oracle(cfg, weights, ids, scaled_and_capped=False)
        assert (want - halves).abs().max() > 0.05 * want.abs().max(), "the pairing was meant to matter"
        model = ei.load_model(folder, dtype=dtype)
        session = ei.Session(model, max_tokens=512, max_seqs=2)
        slot = session.begin()
        rows = [session.step([(slot, ids[:270], list(range(270)))])]
        rows += [session.step([(slot, [token], [0])]) for token in ids[270:]]
        assert_close(dtype, torch.cat(rows), want, f"{dtype} neighbouring pairs")
    finally:
        unregister_architecture(ToyNeighbourPairsConfig.architecture)


# ---------------------------------------------------------------------------
# a rotation that covers the first part of every head only
@dataclass(frozen=True)
class PartialRotarySpec:
    kind: str = "toy_partial_rotary"
    theta: float = 1e4
    dim: int = 8              # rotated width; the head may be wider
    max_positions: int = 256


class PartialRotaryTable:
    """`.table` float32 [positions, dim]: the cosines of the dim/2 pairs (i, i + dim/2) of a
    head's first `dim` elements, then the sines; what lies beyond `dim` is not rotated."""

    def __init__(self, spec, device):
        angle = plain.rope_angles(list(range(spec.max_positions)), spec.dim, spec.theta)
        self.table = torch.cat([torch.cos(angle), torch.sin(angle)], dim=1).float().to(device)
        self.max_positions = spec.max_positions


def partial_rope(x, positions, spec):
    rotated = plain.rope(x[..., :spec.dim], positions, spec.theta)
    return torch.cat([rotated, x[..., spec.dim:].double()], dim=-1)


@pytest.mark.parametrize("dtype,head_dim,rotated", [
    ("float32", 16, 8), ("float32", 48, 12), ("float32", 32, 32), ("bfloat16", 128, 64),
    ("bfloat16", 64, 16), ("bfloat16", 128, 100)])
def test_a_rotation_of_part_of_the_head(dtype, head_dim, rotated):
    """The norm-rotate-store kernel (vector and scalar form) and, in bfloat16 at head sizes 64
    and 128, the decode kernel that does that work itself, with a table narrower than the
    head: whole prompts of unequal lengths, then token by token."""
    from edge_infer_amd.engine import DecoderModel, Session
    from edge_infer_amd.parts import register_position, unregister
    register_position("toy_partial_rotary", PartialRotaryTable)
    try:
        position = PartialRotarySpec(dim=rotated)
        mixer = attention_spec(n_heads=4, n_kv_heads=2, head_dim=head_dim, position=position)
        spec = one_layer_spec(mixer, mlp_spec(), hidden=64)
        params = random_params(spec, 12)
        if dtype == "bfloat16":
            params = {k: v.to(torch.bfloat16).float() for k, v in params.items()}
        model = DecoderModel(spec, params, dtype, DEV)
        session = Session(model, max_tokens=512, max_seqs=2)
        assert model.layers[0].mixer.position.table.shape == (256, rotated)

        def oracle(ids):
            S = len(ids)
            p = "layers.0."
            x = plain.embedding(ids, params["embed.weight"])
            h = plain.rms_norm(x, params[p + "norm1.weight"], 1e-5)
            q = plain.linear(h, params[p + "mixer.q_proj.weight"]).reshape(S, 4, head_dim)
            k = plain.linear(h, params[p + "mixer.k_proj.weight"]).reshape(S, 2, head_dim)
            v = plain.linear(h, params[p + "mixer.v_proj.weight"]).reshape(S, 2, head_dim)
            q = partial_rope(plain.rms_norm(q, params[p + "mixer.q_norm.weight"], 1e-5), range(S), position)
            k = partial_rope(plain.rms_norm(k, params[p + "mixer.k_norm.weight"], 1e-5), range(S), position)
            x = x + plain.linear(plain.attention(q, k, v).reshape(S, -1), params[p + "mixer.o_proj.weight"])
            h = plain.rms_norm(x, params[p + "norm2.weight"], 1e-5)
            x = x + plain.linear(plain.swiglu(plain.linear(h, params[p + "ffn.gate_proj.weight"]),
                                              plain.linear(h, params[p + "ffn.up_proj.weight"])),
                                 params[p + "ffn.down_proj.weight"])
            return plain.linear(plain.rms_norm(x, params["final_norm.weight"], 1e-5), params["head.weight"])

        a, b = random_ids(spec.vocab_size, 90, 1), random_ids(spec.vocab_size, 31, 2)
        ref_a, ref_b = oracle(a), oracle(b)
        # the rotation matters: the same model rotated over the whole head gives other logits
        if rotated < head_dim:
            whole = PartialRotarySpec(dim=head_dim)
            assert (partial_rope(torch.ones(3, 1, head_dim), [5, 6, 7], whole)
                    - partial_rope(torch.ones(3, 1, head_dim), [5, 6, 7], position)).abs().max() > 0.1
        sa, sb = session.begin(), session.begin()
        first = session.step([(sa, a[:70], list(range(70))), (sb, b[:11], list(range(11)))])
        got_a, got_b = [first[:70]], [first[70:]]
        for t in range(20):
            out = session.step([(sa, [a[70 + t]], [0]), (sb, [b[11 + t]], [0])])
            got_a.append(out[:1])
            got_b.append(out[1:])
        assert_close(dtype, torch.cat(got_a), ref_a, f"{dtype} d{head_dim} r{rotated} a")
        assert_close(dtype, torch.cat(got_b), ref_b, f"{dtype} d{head_dim} r{rotated} b")
        if dtype == "bfloat16":
            assert model.layers[0].mixer.matrix_cores and session.graph_replays > 0
    finally:
        unregister("position", "toy_partial_rotary")


def test_a_rotation_table_wider_than_the_head_is_refused():
    from edge_infer_amd.csrc import lib
    from edge_infer_amd.csrc.lib import KernelError
    qkv = torch.zeros(2, 4 * 16, device=DEV)
    table = torch.zeros(8, 24, device=DEV)
    with pytest.raises(KernelError, match="at most head_dim"):
        lib.qk_norm_rope_store(qkv, None, None, 1e-6, table, torch.zeros(2, dtype=torch.int32, device=DEV),
                               torch.zeros(2, dtype=torch.int32, device=DEV),
                               torch.zeros(1, 1, dtype=torch.int32, device=DEV),
                               torch.zeros(2, 2 * 16, device=DEV), torch.zeros(1, 1, 64, 16, device=DEV),
                               torch.zeros(1, 1, 64, 16, device=DEV), 2, 1, 16)


# ---------------------------------------------------------------------------
# a mixer whose cached values are narrower than its keys
@dataclass(frozen=True)
class NarrowValueSpec:
    kind: str = "toy_narrow_values"
    key_dim: int = 12
    value_dim: int = 5


class NarrowValueMixer:
    """One head of causal attention whose keys are `key_dim` wide and whose values `value_dim`:
    its cache pages have those two widths.  Written with library calls on the pages."""

    @classmethod
    def parameters(cls, spec, hidden):
        from edge_infer_amd.weights import ParamSpec
        return {"q.weight": ParamSpec((spec.key_dim, hidden)), "k.weight": ParamSpec((spec.key_dim, hidden)),
                "v.weight": ParamSpec((spec.value_dim, hidden)), "o.weight": ParamSpec((hidden, spec.value_dim))}

    @classmethod
    def cache_request(cls, spec):
        from edge_infer_amd.parts import KVRequest
        return KVRequest(n_kv_heads=1, head_dim=spec.key_dim, value_dim=spec.value_dim)

    def __init__(self, spec, hidden, params, dtype, device, positions):
        self.spec = spec
        self.w = {k: v.to(device=device, dtype=torch.float32) for k, v in params.items()}

    def forward(self, ctx, x, entry):
        group, k_pages, v_pages = ctx.cache.kv(entry.cache)
        assert k_pages.shape[-1] == self.spec.key_dim and v_pages.shape[-1] == self.spec.value_dim
        x = x.float()
        out = torch.empty(x.shape[0], self.spec.value_dim, device=x.device)
        for index, seq in enumerate(ctx.sequences):
            rows = slice(seq.row0, seq.row0 + seq.count)
            pages = ctx.meta.page_table(group)[index].long()
            place = torch.arange(seq.start, seq.start + seq.count, device=x.device)
            k_pages[pages[place // 64], 0, place % 64] = (x[rows] @ self.w["k.weight"].t()).to(k_pages.dtype)
            v_pages[pages[place // 64], 0, place % 64] = (x[rows] @ self.w["v.weight"].t()).to(v_pages.dtype)
            every = torch.arange(seq.start + seq.count, device=x.device)
            keys = k_pages[pages[every // 64], 0, every % 64].float()
            values = v_pages[pages[every // 64], 0, every % 64].float()
            scores = (x[rows] @ self.w["q.weight"].t()) @ keys.t() / math.sqrt(self.spec.key_dim)
            scores = scores.masked_fill(every[None, :] > place[:, None], float("-inf"))
            out[rows] = torch.softmax(scores, dim=-1) @ values
        return out @ self.w["o.weight"].t()


def test_a_cache_whose_values_are_narrower_than_its_keys():
    from edge_infer_amd.parts import register_mixer, unregister
    register_mixer("toy_narrow_values", NarrowValueMixer)
    try:
        mixer = NarrowValueSpec()
        spec = one_layer_spec(mixer, mlp_spec())
        params = random_params(spec, 14)
        model, session = make_session(spec, params, max_tokens=256, max_seqs=2)
        assert session.cache.kv_k[0].shape[-1] == 12 and session.cache.kv_v[0].shape[-1] == 5

        def oracle(ids):
            S = len(ids)
            p = "layers.0."
            x = plain.embedding(ids, params["embed.weight"])
            h = plain.rms_norm(x, params[p + "norm1.weight"], 1e-5)
            q = plain.linear(h, params[p + "mixer.q.weight"])
            k = plain.linear(h, params[p + "mixer.k.weight"])
            v = plain.linear(h, params[p + "mixer.v.weight"])
            scores = (q @ k.t()) / math.sqrt(mixer.key_dim)
            scores = scores.masked_fill(torch.ones(S, S, dtype=torch.bool).triu(1), float("-inf"))
            x = x + plain.linear(torch.softmax(scores, dim=-1) @ v, params[p + "mixer.o.weight"])
            h = plain.rms_norm(x, params[p + "norm2.weight"], 1e-5)
            x = x + plain.linear(plain.swiglu(plain.linear(h, params[p + "ffn.gate_proj.weight"]),
                                              plain.linear(h, params[p + "ffn.up_proj.weight"])),
                                 params[p + "ffn.down_proj.weight"])
            return plain.linear(plain.rms_norm(x, params["final_norm.weight"], 1e-5), params["head.weight"])

        ids = random_ids(spec.vocab_size, 100, 3)
        slot = session.begin()
        rows = [session.step([(slot, ids[:80], list(range(80)))])]
        rows += [session.step([(slot, [token], [0])]) for token in ids[80:]]
        assert_close_f32(torch.cat(rows), oracle(ids), "values narrower than keys")
    finally:
        unregister("mixer", "toy_narrow_values")


def test_an_item_larger_than_a_block_takes_is_refused_before_the_launch():
    """The matrix-core prefill kernel gives a block's waves fixed rows of a work item; the
    binding checks the list's largest item on the host."""
    from edge_infer_amd.csrc import lib
    from edge_infer_amd.csrc.lib import KernelError
    n, heads, kv_heads, d = 300, 4, 2, 64
    q = torch.zeros(n, heads * d, dtype=torch.bfloat16, device=DEV)
    pages = torch.zeros(8, kv_heads, 64, d, dtype=torch.bfloat16, device=DEV)
    capacity = lib.attention_prefill_mfma_positions(heads // kv_heads)
    items = torch.tensor([[0], [0], [capacity + 1]], dtype=torch.int32, device=DEV)
    args = (q, pages, pages.clone(), items[0], items[1], items[2], 1,
            torch.arange(n, dtype=torch.int32, device=DEV),
            torch.arange(8, dtype=torch.int32, device=DEV).reshape(1, 8), torch.empty_like(q),
            heads, kv_heads, d)
    with pytest.raises(KernelError, match="at most"):
        lib.attention_prefill_mfma(*args, largest_item=capacity + 1)
    with pytest.raises(KernelError, match="at most"):
        lib.attention_prefill_mfma(*args)          # looked up on the device
