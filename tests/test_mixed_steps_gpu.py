"""Steps that hold sequences in the middle of decoding beside a newcomer's prompt.

The reference interleaves prefills and decodes of distinct sessions over one model to expose
aliasing of cached keys and values (tools/validation/qwen3_reference.py:396-404,
runtime/tests/qwen3_session_test.cpp:746-839).  This engine's step function takes such a
mixture in one step: entries that bring one token at a position beyond zero beside entries
that bring a whole prompt, or a portion of one.  One schedule runs through `Session.step` and,
as the same lines of JSON, through `bin/trace_run`; every returned row is compared with the
plain implementation, in float32 and in bfloat16, for the two tiny configurations and for a
model of head size 128, whose bfloat16 steps take the matrix-core attention kernels.
"""
import json
import subprocess
import sys
from pathlib import Path

import numpy as np
import pytest
import torch

import plain_qwen3 as plain
from helpers import (BF16_LONG_MAX_REL, BF16_MAX_REL, CONFIGS, LONG, assert_close, assert_close_long, make_folder,
                     make_long_folder, random_ids)

pytestmark = pytest.mark.gpu
ROOT = Path(__file__).resolve().parents[1]
DTYPES = ["float32", "bfloat16"]
# request lengths: r0 and r1 start together; r2 joins whole while they decode; r3 joins in
# three portions, the middle one two tokens across a page boundary (positions 63 and 64);
# r4 takes the slot that r1 gave back
LENGTHS = {"A": [70, 41, 66, 100, 37], "B": [130, 64, 35, 150, 90], "long": [700, 130, 1100, 300, 450]}


def schedule(lengths):
    """[(entries, ended)] with entries (request, first token, one past the last, wanted places
    of the request): the steps of the module's docstring."""
    steps = []
    at = {}

    def advance(request, count, want="last"):
        start = at.get(request, 0)
        at[request] = start + count
        assert count >= 1 and at[request] <= lengths[request], "the schedule outruns a request"
        places = list(range(start, start + count)) if want == "all" else \
            [start + count - 1] if want == "last" else []
        return (request, start, start + count, places)

    tail = 24                                   # tokens every request decodes one by one
    steps.append(([advance(0, lengths[0] - tail - 8), advance(1, lengths[1] - tail - 4)], []))
    for _ in range(3):
        steps.append(([advance(0, 1), advance(1, 1)], []))
    # a whole new prompt beside two decoding sequences; every row of the newcomer is wanted
    steps.append(([advance(0, 1), advance(2, lengths[2] - tail - 6, "all"), advance(1, 1)], []))
    # a prompt's portions beside three decoding sequences
    steps.append(([advance(0, 1), advance(1, 1), advance(2, 1), advance(3, 63, "all")], []))
    steps.append(([advance(3, 2, "all"), advance(0, 1), advance(1, 1, "none"), advance(2, 1)], []))
    steps.append(([advance(0, 1), advance(1, 1), advance(2, 1),
                   advance(3, lengths[3] - tail - 65)], []))
    # r1 decodes to its end and leaves; its slot is the next one handed out
    while at[1] < lengths[1]:
        steps.append(([advance(r, 1) for r in (0, 1, 2, 3)], []))
    steps[-1] = (steps[-1][0], [1])
    steps.append(([advance(0, 1), advance(4, lengths[4] - tail, "all"), advance(2, 1),
                   advance(3, 1)], []))
    # all decoding together until each has brought all its tokens
    while any(at[r] < lengths[r] for r in (0, 2, 3, 4)):
        live = [r for r in (0, 2, 3, 4) if at[r] < lengths[r]]
        entries = [advance(r, 1) for r in live]
        steps.append((entries, [r for r in live if at[r] == lengths[r]]))
    return steps


def fixture_for(which, root):
    if which == "long":
        folder = make_long_folder(root)
        vocab = LONG["vocab_size"]
    else:
        folder = make_folder(which, root)
        vocab = CONFIGS[which]["vocab_size"]
    requests = [random_ids(vocab, n, 300 + i) for i, n in enumerate(LENGTHS[which])]
    cfg, weights = plain.read_folder(folder)
    refs = [plain.forward(weights, cfg, ids) for ids in requests]
    return folder, requests, refs


@pytest.fixture(scope="module")
def fixtures(tmp_path_factory):
    held = {}

    def get(which):
        if which not in held:
            held[which] = fixture_for(which, tmp_path_factory.mktemp(f"mixed_{which}"))
        return held[which]
    return get


def expected_rows(refs, entries):
    rows = [refs[request][place] for request, _, _, places in entries for place in places]
    return torch.stack(rows) if rows else None


class Collected:
    """The rows a schedule returned.  In float32 every step is compared as it comes.  A step of
    this schedule returns one to four rows, and the root-mean-square bound of bfloat16 is
    made for sets of many rows (a single row's error scatters around it), so in bfloat16 a
    step's rows are held to the bound on the largest error only, and all rows of a request
    together to both bounds, as in the other tests of the engine."""

    def __init__(self, dtype, close, refs, what):
        self.dtype, self.close, self.refs, self.what = dtype, close, refs, what
        self.max_rel = BF16_LONG_MAX_REL if close is assert_close_long else BF16_MAX_REL
        self.rows = {}

    def step(self, number, entries, logits):
        want = expected_rows(self.refs, entries)
        if want is None:
            assert logits.shape[0] == 0
            return
        what = f"{self.what} step {number} {[(r, a, b) for r, a, b, _ in entries]}"
        if self.dtype == "float32":
            self.close(self.dtype, logits, want, what)
        else:
            got, want = logits.double().cpu(), want.double()
            assert logits.shape == want.shape
            assert (got - want).abs().max() <= self.max_rel * want.abs().max(), what
        index = 0
        for request, _, _, places in entries:
            for place in places:
                self.rows.setdefault(request, []).append((place, logits[index].clone()))
                index += 1

    def finish(self):
        for request, rows in self.rows.items():
            places = [place for place, _ in rows]
            self.close(self.dtype, torch.stack([row for _, row in rows]).cpu(),
                       self.refs[request][places], f"{self.what} request {request}")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("which", ["A", "B", "long"])
def test_decoding_sequences_and_a_newcomer_in_one_step(fixtures, which, dtype):
    import edge_infer_amd as ei
    folder, requests, refs = fixtures(which)
    close = assert_close_long if which == "long" else assert_close
    steps = schedule(LENGTHS[which])
    model = ei.load_model(folder, dtype=dtype)
    # four slots for five requests: the last one must take a slot that was given back
    session = ei.Session(model, max_tokens=sum((n + 63) // 64 * 64 for n in LENGTHS[which]),
                         max_seqs=4)
    for tensor in session.cache.kv_k + session.cache.kv_v:
        tensor.fill_(float("nan"))            # a key read from a page nobody wrote shows
    slots, freed = {}, []
    mixed = 0
    collected = Collected(dtype, close, refs, f"{which} {dtype}")
    for number, (entries, ended) in enumerate(steps):
        for request, start, _, _ in entries:
            if request not in slots:
                assert start == 0
                slots[request] = session.begin()
                if request == 4:
                    assert slots[4] == freed[-1], "the newcomer was meant to reuse a slot"
        counts = [stop - start for _, start, stop, _ in entries]
        mixed += min(counts) == 1 and max(counts) > 1
        logits = session.step([(slots[request], requests[request][start:stop],
                                [place - start for place in places])
                               for request, start, stop, places in entries])
        collected.step(number, entries, logits)
        for request in ended:
            freed.append(slots[request])
            session.end(slots.pop(request))
    collected.finish()
    assert mixed >= 5 and not slots
    assert session.graph_replays > 0          # the all-decode steps ran from graphs


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("which", ["B", "long"])
def test_the_same_schedule_through_trace_replay(fixtures, tmp_path, which, dtype):
    folder, requests, refs = fixtures(which)
    close = assert_close_long if which == "long" else assert_close
    steps = schedule(LENGTHS[which])
    lines = []
    for number, (entries, ended) in enumerate(steps):
        lines.append(json.dumps({
            "step": number,
            "entries": [{"id": f"r{request}", "tokens": requests[request][start:stop],
                         "want": [place - start for place in places]}
                        for request, start, stop, places in entries],
            "end": [f"r{request}" for request in ended]}))
    out_dir = tmp_path / "out"
    run = subprocess.run([sys.executable, str(ROOT / "bin" / "trace_run"), "--model", str(folder),
                          "--dtype", dtype, "--out", str(out_dir), "--max-tokens",
                          str(sum((n + 63) // 64 * 64 for n in LENGTHS[which]))],
                         input="\n".join(lines) + "\n", capture_output=True, text=True, timeout=600)
    assert run.returncode == 0, run.stderr[-2000:]
    vocab = refs[0].shape[1]
    collected = Collected(dtype, close, refs, f"replayed {which} {dtype}")
    for number, (entries, _) in enumerate(steps):
        path = out_dir / f"{number}.f32"
        if expected_rows(refs, entries) is None:
            assert not path.exists()
            continue
        got = torch.from_numpy(np.fromfile(str(path), dtype="<f4").reshape(-1, vocab).copy())
        collected.step(number, entries, got)
    collected.finish()


@pytest.mark.parametrize("dtype", DTYPES)
def test_two_sessions_of_one_model_interleaved(fixtures, dtype):
    """The reference's own schedule: sessions over shared weights take turns, a prefill of
    one between the decode steps of another."""
    import edge_infer_amd as ei
    folder, requests, refs = fixtures("B")
    model = ei.load_model(folder, dtype=dtype)
    sessions = [ei.Session(model, max_tokens=256, max_seqs=1) for _ in range(3)]
    slots = [session.begin() for session in sessions]
    cuts = [len(requests[i]) - 10 for i in range(3)]
    got = [[] for _ in range(3)]
    got[0].append(sessions[0].step([(slots[0], requests[0][:cuts[0]], [cuts[0] - 1])]))
    for t in range(10):
        if t == 2:     # the second session's prompt comes between the first one's decode steps
            got[1].append(sessions[1].step([(slots[1], requests[1][:cuts[1]], [cuts[1] - 1])]))
        if t == 5:
            got[2].append(sessions[2].step([(slots[2], requests[2][:cuts[2]], [cuts[2] - 1])]))
        for i in range(3):
            first = (0, 2, 5)[i]
            if t >= first:
                token = requests[i][cuts[i] + t - first]
                got[i].append(sessions[i].step([(slots[i], [token], [0])]))
    for i in range(3):
        rows = torch.cat(got[i])
        assert_close(dtype, rows, refs[i][cuts[i] - 1:cuts[i] - 1 + rows.shape[0]],
                     f"{dtype} session {i}")


# ---------------------------------------------------------------------------
# Schedules nobody thought of: drawn from a seeded generator
def random_schedule(seed, max_seqs, longest, n_requests=14, n_steps=70):
    """(lengths, steps): requests of random lengths begin whenever a slot is free, each step
    takes one token or a portion of 2 to 70 tokens of some of the live requests (the others
    sit the step out), wants the last row, all rows, none or a few of them, and requests leave
    when their tokens are used up or, now and then, earlier.  Every step mixes what it likes."""
    import random
    rng = random.Random(seed)
    lengths, steps = [], []
    at = {}                                                    # live request -> tokens brought
    while len(steps) < n_steps and (at or len(lengths) < n_requests):
        while len(at) < max_seqs and len(lengths) < n_requests and (not at or rng.random() < 0.3):
            lengths.append(rng.choice([n for n in (2, 3, 17, 63, 64, 65, 66, 100, 128, 129, 190, 257)
                                       if n <= longest]))
            at[len(lengths) - 1] = 0
        entries, ended = [], []
        for request in sorted(at, key=lambda r: rng.random()):     # entries in any order
            left = lengths[request] - at[request]
            if entries and rng.random() < 0.15:
                continue                                           # sits this step out
            count = 1
            if left >= 2 and (at[request] == 0 or rng.random() < 0.3):
                count = rng.randint(2, min(left, 70))
            start = at[request]
            choice = rng.random()
            if choice < 0.5:
                places = [start + count - 1]
            elif choice < 0.7:
                places = list(range(start, start + count))
            elif choice < 0.8:
                places = []
            else:
                places = sorted(rng.sample(range(start, start + count), min(count, 3)))
            entries.append((request, start, start + count, places))
            at[request] += count
            if at[request] == lengths[request] or rng.random() < 0.02:
                ended.append(request)
        for request in ended:
            del at[request]
        steps.append((entries, ended))
    return lengths, steps


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("which,seed", [("A", 1), ("B", 2), ("long", 3), ("B", 4)])
def test_schedules_drawn_at_random(tmp_path, which, seed, dtype):
    """Every row that a drawn schedule returns against the plain implementation: slots are
    given back and taken again in any order, sequences idle, prompts come in portions of any
    size beside decoding sequences.  The cache starts full of NaN."""
    import edge_infer_amd as ei
    max_seqs = 5
    shape = LONG if which == "long" else CONFIGS[which]
    lengths, steps = random_schedule(seed, max_seqs, min(257, shape["max_position_embeddings"]))
    assert len(lengths) >= 10 and any(ended for _, ended in steps)
    vocab = shape["vocab_size"]
    if which == "long":
        folder, close = make_long_folder(tmp_path), assert_close_long
    else:
        folder, close = make_folder(which, tmp_path), assert_close
    requests = [random_ids(vocab, n, 900 + 31 * seed + i) for i, n in enumerate(lengths)]
    cfg, weights = plain.read_folder(folder)
    refs = [plain.forward(weights, cfg, ids) for ids in requests]
    session = ei.Session(ei.load_model(folder, dtype=dtype), max_tokens=max_seqs * 320,
                         max_seqs=max_seqs)
    for tensor in session.cache.kv_k + session.cache.kv_v:
        tensor.fill_(float("nan"))
    slots, seen_slots = {}, []
    collected = Collected(dtype, close, refs, f"drawn {which} {seed} {dtype}")
    for number, (entries, ended) in enumerate(steps):
        for request, start, _, _ in entries:
            if request not in slots:
                assert start == 0
                slots[request] = session.begin()
                seen_slots.append(slots[request])
        logits = session.step([(slots[request], requests[request][start:stop],
                                [place - start for place in places])
                               for request, start, stop, places in entries])
        collected.step(number, entries, logits)
        for request in ended:
            session.end(slots.pop(request))
    collected.finish()
    for slot in slots.values():
        session.end(slot)
    assert len(set(seen_slots)) <= max_seqs < len(seen_slots), "slots were meant to be used again"
