"""State of fixed size per sequence as a first-class part of the cache: a toy mixer, defined
here and nowhere in the framework, that finds its state row on the device through the
step's `seq_slot` section, runs from captured graphs, and survives a failed step (the state
it had updated in place is put back, so the retried step gives the right logits)."""
from dataclasses import dataclass

import pytest
import torch

import plain_qwen3 as plain
from helpers import assert_close_f32
from test_parts_gpu import attention_spec, make_session, mlp_spec, random_params

pytestmark = pytest.mark.gpu

HIDDEN, VOCAB = 48, 61


@dataclass(frozen=True)
class DecaySpec:
    kind: str = "toy_device_decay"
    decay: float = 0.85
    width: int = HIDDEN


class DeviceDecayMixer:
    """state <- decay * state + W x;  y = state.  Everything happens on the device with
    tensors of fixed shape, so a decode step can be captured: the state row of a sequence is
    `seq_slot[row_seq[row]]`, padding points at the spare row."""

    capture_safe = True
    fail_once = False        # the test's switch: raise after the state has been updated

    @classmethod
    def parameters(cls, spec, hidden):
        from edge_infer_amd.weights import ParamSpec
        return {"in_proj.weight": ParamSpec((spec.width, hidden))}

    @classmethod
    def cache_request(cls, spec):
        from edge_infer_amd.parts import StateRequest
        return StateRequest(shape=(spec.width,))

    def __init__(self, spec, hidden, params, dtype, device, positions):
        from edge_infer_amd.parts import Linear
        self.decay = spec.decay
        self.proj = Linear(params["in_proj.weight"], dtype, device)

    def forward(self, ctx, x, entry):
        meta = ctx.meta
        state = ctx.cache.state(entry.cache)                  # [slots + 1, width] float32
        u = self.proj.forward(ctx, x, "toy.u")                # float32 [rows, width]
        row_seq = meta.row_seq.long()
        valid = row_seq >= 0
        seq = row_seq.clamp(min=0)
        slot = meta.seq_slot.long()
        carried = state.index_select(0, slot).index_select(0, seq)
        pos = meta.row_pos
        since = (pos - meta.seq_start.index_select(0, seq) + 1).float()
        gap = pos[:, None] - pos[None, :]
        together = (row_seq[:, None] == row_seq[None, :]) & valid[:, None] & (gap >= 0)
        weight = torch.where(together, self.decay ** gap.clamp(min=0).float(), 0.0)
        out = (weight[:, :, None] * u[None, :, :]).sum(1) + (self.decay ** since)[:, None] * carried
        out = torch.where(valid[:, None], out, 0.0)
        if entry.writes_cache:
            last = (torch.cumsum(meta.seq_count, 0) - 1).clamp(min=0).long()
            state.index_copy_(0, slot, out.index_select(0, last))
        if type(self).fail_once and entry.cache == 2:
            type(self).fail_once = False
            raise RuntimeError("forced failure after the state was updated")
        return out


@pytest.fixture()
def toy():
    from edge_infer_amd.config.specs import LayerSpec, ModelSpec, NormSpec, ScheduleEntry
    from edge_infer_amd.parts import register_mixer, unregister
    register_mixer("toy_device_decay", DeviceDecayMixer)
    norm = NormSpec(eps=1e-5)
    layers = (LayerSpec("prenorm", norm, attention_spec(), mlp_spec()),
              LayerSpec("prenorm", norm, DecaySpec(), mlp_spec(56)))
    # the toy layer runs twice, each run with a state entry of its own
    schedule = (ScheduleEntry(0, 0), ScheduleEntry(1, 1), ScheduleEntry(1, 2))
    spec = ModelSpec(architecture="ToyStateForCausalLM", vocab_size=VOCAB, hidden_size=HIDDEN,
                     layers=layers, schedule=schedule, final_norm=norm, tie_word_embeddings=False,
                     max_position_embeddings=256, bos_token_id=0, eos_token_id=1)
    params = random_params(spec, 4)

    def oracle(ids):
        S = len(ids)
        x = plain.embedding(ids, params["embed.weight"])
        for entry in schedule:
            p = f"layers.{entry.layer}."
            h = plain.rms_norm(x, params[p + "norm1.weight"], 1e-5)
            if entry.layer == 0:
                m = layers[0].mixer
                q, k, v = (plain.linear(h, params[p + f"mixer.{n}_proj.weight"]).reshape(S, heads, m.head_dim)
                           for n, heads in (("q", m.n_heads), ("k", m.n_kv_heads), ("v", m.n_kv_heads)))
                q = plain.rope(plain.rms_norm(q, params[p + "mixer.q_norm.weight"], m.qk_norm_eps),
                               list(range(S)), m.position.theta)
                k = plain.rope(plain.rms_norm(k, params[p + "mixer.k_norm.weight"], m.qk_norm_eps),
                               list(range(S)), m.position.theta)
                mixed = plain.linear(plain.attention(q, k, v).reshape(S, -1),
                                     params[p + "mixer.o_proj.weight"])
            else:
                u = plain.linear(h, params[p + "mixer.in_proj.weight"])
                s, rows = torch.zeros(HIDDEN, dtype=torch.float64), []
                for r in range(S):
                    s = layers[1].mixer.decay * s + u[r]
                    rows.append(s)
                mixed = torch.stack(rows)
            x = x + mixed
            h = plain.rms_norm(x, params[p + "norm2.weight"], 1e-5)
            x = x + plain.linear(plain.swiglu(plain.linear(h, params[p + "ffn.gate_proj.weight"]),
                                              plain.linear(h, params[p + "ffn.up_proj.weight"])),
                                 params[p + "ffn.down_proj.weight"])
        return plain.linear(plain.rms_norm(x, params["final_norm.weight"], 1e-5), params["head.weight"])

    try:
        yield spec, params, oracle
    finally:
        DeviceDecayMixer.fail_once = False
        unregister("mixer", "toy_device_decay")


def sequences():
    g = torch.Generator().manual_seed(3)
    return [torch.randint(0, VOCAB, (n,), generator=g).tolist() for n in (70, 31, 45)]


def test_a_stateful_mixer_runs_from_captured_graphs(toy):
    """Three sequences of unequal length decode together from a graph; the shortest ends
    early, so later replays run with a padding row whose state is the spare row; every
    replay is compared with the plain recomputation, with eager work in between."""
    spec, params, oracle = toy
    model, session = make_session(spec, params, max_tokens=1024, max_seqs=3)
    assert session.graphs and model.capture_safe()
    assert session.cache.states[0].shape == (2, 3 + 1, HIDDEN)
    a, b, c = sequences()
    refs = [oracle(ids) for ids in (a, b, c)]
    cuts = [50, 20, 30]
    slots = [session.begin() for _ in range(3)]
    out = session.step([(s, ids[:cut], [cut - 1]) for s, ids, cut in zip(slots, (a, b, c), cuts)])
    got = [[row] for row in out]
    live = [0, 1, 2]
    for t in range(15):
        live = [i for i in live if cuts[i] + t < len((a, b, c)[i])]
        out = session.step([(slots[i], [(a, b, c)[i][cuts[i] + t]], [0]) for i in live])
        for i, row in zip(live, out):
            got[i].append(row)
        torch.cuda.synchronize()
        _ = torch.ones(1000, device="cuda").sum().item()      # eager work between replays
    for i in range(3):
        rows = torch.stack(got[i])
        assert_close_f32(rows, refs[i][cuts[i] - 1:cuts[i] - 1 + len(rows)], f"sequence {i}")
    assert session.graph_replays >= 10 and session.graph_captures >= 1
    # a slot that is used again starts from zero state
    session.end(slots[1])
    again = session.begin()
    assert again == slots[1]
    out = session.step([(again, c[:9], [8])])
    assert_close_f32(out, refs[2][8:9], "a reused slot")


@pytest.mark.parametrize("graphs", [False, True])
def test_a_failed_step_puts_the_state_back(toy, graphs):
    """The mixer raises after both of its runs have updated their state in place.  The
    session keeps the lengths it had and restores the state rows of the step's slots, so the
    same step again gives the logits of a run that never failed; a sequence that was not in
    the failed step is untouched."""
    spec, params, oracle = toy
    from edge_infer_amd.engine import Session
    model, _ = make_session(spec, params)
    session = Session(model, max_tokens=1024, max_seqs=3, graphs=graphs)
    a, b, c = sequences()
    ref_a, ref_b, ref_c = oracle(a), oracle(b), oracle(c)
    sa, sb, sc = session.begin(), session.begin(), session.begin()
    session.step([(sc, c[:10], [])])
    # a prompt step fails
    DeviceDecayMixer.fail_once = True
    with pytest.raises(RuntimeError, match="forced failure"):
        session.step([(sa, a[:40], [39]), (sb, b[:12], [11])])
    assert session.length(sa) == 0 and session.length(sb) == 0 and session.length(sc) == 10
    out = session.step([(sa, a[:40], [39]), (sb, b[:12], [11])])
    assert_close_f32(out, torch.stack([ref_a[39], ref_b[11]]), "the prompt step again")
    # a decode step fails (with graphs: the eager run before the capture)
    DeviceDecayMixer.fail_once = True
    with pytest.raises(RuntimeError, match="forced failure"):
        session.step([(sa, [a[40]], [0]), (sb, [b[12]], [0])])
    assert session.length(sa) == 40
    rows_a, rows_b = [], []
    for t in range(6):
        out = session.step([(sa, [a[40 + t]], [0]), (sb, [b[12 + t]], [0])])
        rows_a.append(out[0])
        rows_b.append(out[1])
    assert_close_f32(torch.stack(rows_a), ref_a[40:46], "decoding after the failed step")
    assert_close_f32(torch.stack(rows_b), ref_b[12:18], "decoding after the failed step")
    assert session.graph_replays > 0 if graphs else session.graph_replays == 0
    out = session.step([(sc, c[10:], [len(c) - 11])])
    assert_close_f32(out, ref_c[-1:], "the sequence that was not in the failed steps")
