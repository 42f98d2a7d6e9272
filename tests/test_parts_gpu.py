"""Each part alone against its plain reference, and a toy mixer with state of its own
that is registered, built and stepped without a change to the framework's files."""
from dataclasses import dataclass

import pytest
import torch

import plain_qwen3 as plain
from helpers import assert_close_f32

pytestmark = pytest.mark.gpu
DEV = "cuda"


def make_session(spec, params, dtype="float32", max_tokens=512, max_seqs=4):
    from edge_infer_amd.engine import DecoderModel, Session
    model = DecoderModel(spec, params, dtype, DEV)
    return model, Session(model, max_tokens=max_tokens, max_seqs=max_seqs)


def one_layer_spec(mixer, ffn, norm_eps=1e-5, hidden=40, vocab=53, max_pos=256):
    from edge_infer_amd.config.specs import LayerSpec, ModelSpec, NormSpec, default_schedule
    norm = NormSpec(eps=norm_eps)
    return ModelSpec(architecture="test", vocab_size=vocab, hidden_size=hidden,
                     layers=(LayerSpec(block="prenorm", norm=norm, mixer=mixer, feed_forward=ffn),),
                     schedule=default_schedule(1), final_norm=norm, tie_word_embeddings=False,
                     max_position_embeddings=max_pos, bos_token_id=0, eos_token_id=1)


def random_params(spec, seed=0):
    from edge_infer_amd.engine.model import expected_parameters
    from edge_infer_amd.weights import random_parameters
    expected = expected_parameters(spec, lambda path: path)
    params = random_parameters(expected, seed, dtype=torch.float32)
    # N(0, 0.02) matrices make tiny signals; scale the matrices up for a sharper test
    return {k: (v * 8 if v.dim() == 2 else v) for k, v in params.items()}


def context_for(session, seqs_tokens):
    """A step context over fresh slots, without running the model."""
    from edge_infer_amd.engine.batch import SeqStep
    seqs = []
    for start, tokens in seqs_tokens:
        slot = session.begin()
        session.cache.lengths[slot] = start
        seqs.append(SeqStep(slot=slot, start=start, tokens=tokens))
    session.cache.grow([(s.slot, s.start + s.count) for s in seqs])
    return session.context_for(seqs)


def attention_spec(**kw):
    from edge_infer_amd.config.specs import AttentionSpec, PositionSpec
    base = dict(n_heads=6, n_kv_heads=2, head_dim=16, qk_norm=True, qk_norm_eps=1e-5,
                position=PositionSpec(kind="rope", theta=5e4, dim=16, max_positions=256))
    base.update(kw)
    return AttentionSpec(**base)


def mlp_spec(inter=72):
    from edge_infer_amd.config.specs import GatedMLPSpec
    return GatedMLPSpec(intermediate_size=inter)


def test_rotary_table():
    from edge_infer_amd.config.specs import PositionSpec
    from edge_infer_amd.parts import RotaryTable
    table = RotaryTable(PositionSpec(theta=1e6, dim=48, max_positions=300), DEV).table.cpu()
    angle = plain.rope_angles(list(range(300)), 48, 1e6)
    # float32 pow may differ by an ulp between libraries: two ulps of the frequency
    # times the position, plus the rounding of the stored value
    bound = 3e-7 + angle * 2.4e-7
    assert ((table[:, :24].double() - torch.cos(angle)).abs() <= bound).all()
    assert ((table[:, 24:].double() - torch.sin(angle)).abs() <= bound).all()


def test_norm_part():
    from edge_infer_amd.config.specs import NormSpec
    from edge_infer_amd.parts import RMSNorm, Workspace
    from edge_infer_amd.parts.base import StepContext
    weight = 1 + 0.1 * torch.randn(200)
    part = RMSNorm(NormSpec(eps=3e-4), 200, {"weight": weight.to(torch.bfloat16)}, torch.float32, DEV)
    assert part.weight.dtype == torch.float32
    ctx = StepContext(dtype=torch.float32, device=DEV, n_rows=5, n_seqs=1, decode=False, meta=None,
                      cache=None, workspace=Workspace(DEV), max_context=5)
    residual = torch.randn(5, 200, device=DEV)
    delta = torch.randn(5, 200, device=DEV)
    expected = plain.rms_norm(residual.cpu().double() + delta.cpu().double(),
                              weight.to(torch.bfloat16), 3e-4)
    out = part.add_norm(ctx, residual, delta, "h")
    assert_close_f32(out, expected, "norm part")


@pytest.mark.parametrize("variant", ["qwen3", "no_norm_no_rope", "window", "scale"])
def test_attention_part(variant):
    """The mixer alone: whole sequences of unequal lengths, then a chunk appended."""
    from edge_infer_amd.config.specs import PositionSpec
    kw = {}
    if variant == "no_norm_no_rope":
        kw = dict(qk_norm=False, position=PositionSpec(kind="none"))
    elif variant == "window":
        kw = dict(window=9)
    elif variant == "scale":
        kw = dict(scale=0.5, n_heads=4, n_kv_heads=4, head_dim=32,
                  position=PositionSpec(kind="rope", theta=1e4, dim=32, max_positions=256))
    mixer = attention_spec(**kw)
    spec = one_layer_spec(mixer, mlp_spec())
    params = random_params(spec, 3)
    model, session = make_session(spec, params)
    part = model.layers[0].mixer
    from edge_infer_amd.config.specs import ScheduleEntry
    H = spec.hidden_size
    lengths = [70, 9, 130]
    x = torch.randn(sum(lengths), H, device=DEV)

    def plain_mixer(xs):
        S = xs.shape[0]
        p = "layers.0.mixer."
        q = plain.linear(xs, params[p + "q_proj.weight"]).reshape(S, mixer.n_heads, mixer.head_dim)
        k = plain.linear(xs, params[p + "k_proj.weight"]).reshape(S, mixer.n_kv_heads, mixer.head_dim)
        v = plain.linear(xs, params[p + "v_proj.weight"]).reshape(S, mixer.n_kv_heads, mixer.head_dim)
        if mixer.qk_norm:
            q = plain.rms_norm(q, params[p + "q_norm.weight"], mixer.qk_norm_eps)
            k = plain.rms_norm(k, params[p + "k_norm.weight"], mixer.qk_norm_eps)
        if mixer.position.kind == "rope":
            q = plain.rope(q, list(range(S)), mixer.position.theta)
            k = plain.rope(k, list(range(S)), mixer.position.theta)
        if mixer.scale is not None:          # plain.attention scales by 1/sqrt(d)
            q = q * (mixer.scale * mixer.head_dim ** 0.5)
        a = plain.attention(q, k, v, window=mixer.window)
        return plain.linear(a.reshape(S, -1), params[p + "o_proj.weight"])

    # all but the last 5 tokens of each sequence in one step, then the rest as a chunk
    first = [n - 5 for n in lengths]
    ctx, plan = context_for(session, [(0, [0] * n) for n in first])
    rows, at = [], 0
    for n, f in zip(lengths, first):
        rows.append(x[at:at + f])
        at += n
    out = part.forward(ctx, torch.cat(rows).contiguous(), ScheduleEntry(0, 0))
    expected, at = [], 0
    for n, f in zip(lengths, first):
        expected.append(plain_mixer(x[at:at + n].cpu())[:f])
        at += n
    assert_close_f32(out, torch.cat(expected), f"attention part {variant} (prefill)")
    growth = [(s.slot, s.start + s.count) for s in plan.seqs]
    slots = [s.slot for s in plan.seqs]
    session.cache.commit(growth)
    # the chunk: built by hand on the same slots
    from edge_infer_amd.engine.batch import SeqStep
    seqs = [SeqStep(slot=slot, start=f, tokens=[0] * 5) for slot, f in zip(slots, first)]
    session.cache.grow([(s.slot, s.start + 5) for s in seqs])
    ctx, plan = session.context_for(seqs)
    rows, at = [], 0
    for n, f in zip(lengths, first):
        rows.append(x[at + f:at + n])
        at += n
    out = part.forward(ctx, torch.cat(rows).contiguous(), ScheduleEntry(0, 0))
    expected, at = [], 0
    for n, f in zip(lengths, first):
        expected.append(plain_mixer(x[at:at + n].cpu())[f:])
        at += n
    assert_close_f32(out, torch.cat(expected), f"attention part {variant} (chunk)")


def test_feed_forward_part():
    spec = one_layer_spec(attention_spec(), mlp_spec(inter=72))
    params = random_params(spec, 5)
    model, session = make_session(spec, params)
    ctx, _ = context_for(session, [(0, [0] * 11)])
    x = torch.randn(11, spec.hidden_size, device=DEV)
    out = model.layers[0].ffn.forward(ctx, x)
    p = "layers.0.ffn."
    expected = plain.linear(plain.swiglu(plain.linear(x.cpu(), params[p + "gate_proj.weight"]),
                                         plain.linear(x.cpu(), params[p + "up_proj.weight"])),
                            params[p + "down_proj.weight"])
    assert_close_f32(out, expected, "feed-forward part")


# ---------------------------------------------------------------------------
# a toy mixer with state of its own, defined here and nowhere in the framework
@dataclass(frozen=True)
class DecaySpec:
    kind: str = "toy_decay"
    decay: float = 0.9


class DecayMixer:
    """state <- decay * state + W x;  y = state.  One float32 vector per sequence."""

    @classmethod
    def parameters(cls, spec, hidden):
        from edge_infer_amd.weights import ParamSpec
        return {"in_proj.weight": ParamSpec((hidden, hidden))}

    @classmethod
    def cache_request(cls, spec):
        from edge_infer_amd.parts import StateRequest
        return None  # replaced below once the hidden size is known

    def __init__(self, spec, hidden, params, dtype, device, positions):
        self.spec = spec
        self.weight = params["in_proj.weight"].to(device=device, dtype=torch.float32)

    def forward(self, ctx, x, entry):
        state = ctx.cache.state(entry.cache)            # [slots, hidden] float32
        out = torch.empty(x.shape, dtype=torch.float32, device=x.device)
        projected = x.float() @ self.weight.t()
        for seq in ctx.sequences:
            s = state[seq.slot].clone()
            for r in range(seq.row0, seq.row0 + seq.count):
                s = self.spec.decay * s + projected[r]
                out[r] = s
            if entry.writes_cache:
                state[seq.slot] = s
        return out


def test_toy_mixer_with_state_is_registered_built_and_stepped():
    from edge_infer_amd.config import register_architecture, unregister_architecture
    from edge_infer_amd.config.specs import (LayerSpec, ModelSpec, NormSpec, PositionSpec,
                                             ScheduleEntry)
    from edge_infer_amd.parts import StateRequest, register_mixer, unregister

    hidden, vocab = 40, 53
    DecayMixer.cache_request = classmethod(lambda cls, spec: StateRequest(shape=(hidden,)))
    register_mixer("toy_decay", DecayMixer)
    try:
        norm = NormSpec(eps=1e-5)
        layers = (LayerSpec("prenorm", norm, attention_spec(), mlp_spec()),
                  LayerSpec("prenorm", norm, DecaySpec(decay=0.8), mlp_spec(56)),
                  LayerSpec("prenorm", norm, attention_spec(n_heads=2, n_kv_heads=1, head_dim=32,
                                                            position=PositionSpec(kind="none")),
                            mlp_spec()))
        # layer 1 (the toy) runs twice, each run with state of its own; the last run of
        # layer 0 reads the cache that its first run wrote
        schedule = (ScheduleEntry(0, 0), ScheduleEntry(1, 1), ScheduleEntry(2, 2),
                    ScheduleEntry(1, 3), ScheduleEntry(0, 0, writes_cache=False))
        spec = ModelSpec(architecture="ToyForCausalLM", vocab_size=vocab, hidden_size=hidden,
                         layers=layers, schedule=schedule, final_norm=norm,
                         tie_word_embeddings=False, max_position_embeddings=256, bos_token_id=0,
                         eos_token_id=1)
        params = random_params(spec, 9)
        model, session = make_session(spec, params, max_tokens=1024, max_seqs=3)
        layout = session.cache.layout
        assert len(layout.kv_groups) == 2 and len(layout.state_groups) == 1
        assert layout.state_groups[0][1] == [1, 3]
        assert session.cache.states[0].shape == (2, 3 + 1, hidden)    # one spare row

        def oracle(ids):
            """The same model, whole sequence, float64."""
            S = len(ids)
            x = plain.embedding(ids, params["embed.weight"])

            kept = {}

            def attn(layer, h, mixer, entry):
                p = f"layers.{layer}.mixer."
                q = plain.linear(h, params[p + "q_proj.weight"]).reshape(S, mixer.n_heads, mixer.head_dim)
                k = plain.linear(h, params[p + "k_proj.weight"]).reshape(S, mixer.n_kv_heads, mixer.head_dim)
                v = plain.linear(h, params[p + "v_proj.weight"]).reshape(S, mixer.n_kv_heads, mixer.head_dim)
                q = plain.rms_norm(q, params[p + "q_norm.weight"], mixer.qk_norm_eps)
                k = plain.rms_norm(k, params[p + "k_norm.weight"], mixer.qk_norm_eps)
                if mixer.position.kind == "rope":
                    q = plain.rope(q, list(range(S)), mixer.position.theta)
                    k = plain.rope(k, list(range(S)), mixer.position.theta)
                if entry.writes_cache:
                    kept[entry.cache] = (k, v)
                else:                       # keys and values of the run that wrote the entry
                    k, v = kept[entry.cache]
                return plain.linear(plain.attention(q, k, v).reshape(S, -1), params[p + "o_proj.weight"])

            def decay(layer, h, mixer, entry):
                u = plain.linear(h, params[f"layers.{layer}.mixer.in_proj.weight"])
                s = torch.zeros(hidden, dtype=torch.float64)
                rows = []
                for r in range(S):
                    s = mixer.decay * s + u[r]
                    rows.append(s)
                return torch.stack(rows)

            for entry in schedule:
                layer = layers[entry.layer]
                p = f"layers.{entry.layer}."
                h = plain.rms_norm(x, params[p + "norm1.weight"], 1e-5)
                mix = decay if layer.mixer.kind == "toy_decay" else attn
                x = x + mix(entry.layer, h, layer.mixer, entry)
                h = plain.rms_norm(x, params[p + "norm2.weight"], 1e-5)
                x = x + plain.linear(plain.swiglu(plain.linear(h, params[p + "ffn.gate_proj.weight"]),
                                                  plain.linear(h, params[p + "ffn.up_proj.weight"])),
                                     params[p + "ffn.down_proj.weight"])
            return plain.linear(plain.rms_norm(x, params["final_norm.weight"], 1e-5),
                                params["head.weight"])

        g = torch.Generator().manual_seed(1)
        a = torch.randint(0, vocab, (90,), generator=g).tolist()
        b = torch.randint(0, vocab, (37,), generator=g).tolist()
        ref_a, ref_b = oracle(a), oracle(b)
        # whole, as a batch of two
        sa, sb = session.begin(), session.begin()
        logits = session.step([(sa, a, list(range(90))), (sb, b, list(range(37)))])
        assert_close_f32(logits[:90], ref_a, "toy model whole a")
        assert_close_f32(logits[90:], ref_b, "toy model whole b")
        session.end(sa)
        session.end(sb)
        # a prefix, then token by token: the state carries over, and a reused slot starts at zero
        sb, sa = session.begin(), session.begin()
        rows = [session.step([(sa, a[:60], [59]), (sb, b[:7], [6])])]
        got_a, got_b = [rows[0][0]], [rows[0][1]]
        for t in range(30):
            live = [(sa, [a[60 + t]], [0]), (sb, [b[7 + t]], [0])]
            out = session.step(live)
            got_a.append(out[0])
            got_b.append(out[1])
        assert_close_f32(torch.stack(got_a), ref_a[59:], "toy model decode a")
        assert_close_f32(torch.stack(got_b), ref_b[6:37], "toy model decode b")
        # it is selected through the registry like any architecture
        class ToyConfig:
            @classmethod
            def from_dict(cls, raw):
                return cls()
            def model_spec(self):
                return spec
        register_architecture("ToyForCausalLM", ToyConfig)
        try:
            from edge_infer_amd.config import resolve_architecture
            assert resolve_architecture({"architectures": ["ToyForCausalLM"]}).config_class is ToyConfig
        finally:
            unregister_architecture("ToyForCausalLM")
    finally:
        unregister("mixer", "toy_decay")
