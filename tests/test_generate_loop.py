"""Decisions of the generation loop, with a scripted session and sampler (no GPU)."""
import pytest
import torch

from edge_infer_amd.cache import CacheFull
from edge_infer_amd.engine.generate import Request, generate, plan_batches
from edge_infer_amd.sampling import SamplingParams

VOCAB = 32


class ScriptedSession:
    """Logits that make greedy decoding count upwards from the last token fed:
    the next token after t is (t + 1) mod VOCAB.  Records every step it is given."""

    def __init__(self, capacity=64, max_batch=4, pages=16):
        self.capacity = capacity
        self.max_batch = max_batch
        self.pages = pages
        self.live = {}
        self.next_slot = 0
        self.steps = []
        self.ended = []

    def free_tokens(self):
        return self.pages * 64

    def begin(self):
        if len(self.live) >= self.max_batch:
            raise CacheFull("no slot")
        slot = self.next_slot
        self.next_slot += 1
        self.live[slot] = []
        return slot

    def end(self, slot):
        self.ended.append(slot)
        del self.live[slot]            # KeyError on a double release

    def step(self, entries, copy=True):
        self.steps.append([(slot, list(tokens), list(want)) for slot, tokens, want in entries])
        rows = []
        for slot, tokens, want in entries:
            assert len(self.live[slot]) + len(tokens) <= self.capacity
            for w in want:
                row = torch.zeros(VOCAB)
                row[(tokens[w] + 1) % VOCAB] = 5.0
                rows.append(row)
            self.live[slot].extend(tokens)
        return torch.stack(rows) if rows else torch.zeros(0, VOCAB)


def argmax_sampler(logits, params, streams, counters):
    argmax_sampler.calls.append((list(streams), list(counters)))
    return logits.argmax(dim=-1).tolist()


argmax_sampler.calls = []


def run(session, prompts, **kwargs):
    argmax_sampler.calls = []
    kwargs.setdefault("params", SamplingParams(temperature=0.0))
    return generate(session, argmax_sampler, prompts, vocab_size=VOCAB, **kwargs)


def test_unequal_prompts_one_prefill_then_one_token_each():
    s = ScriptedSession()
    out = run(s, [[1, 2, 3], [10], [20, 21]], max_new_tokens=3)
    assert out == [[4, 5, 6], [11, 12, 13], [22, 23, 24]]
    assert [len(t) for _, t, _ in s.steps[0]] == [3, 1, 2]           # all prompts in one step
    assert [w for _, _, w in s.steps[0]] == [[2], [0], [1]]           # logits at each last row
    assert all(len(t) == 1 for step in s.steps[1:] for _, t, _ in step)
    assert len(s.steps) == 3                                           # 1 prefill + 2 decodes
    assert sorted(s.ended) == [0, 1, 2] and not s.live


def test_max_length_counts_the_prompt():
    s = ScriptedSession()
    out = run(s, [[1, 2, 3, 4]], max_length=6)
    assert out == [[5, 6]]
    s = ScriptedSession()
    assert run(s, [[1, 2, 3, 4]], max_length=4) == [[]]
    assert s.steps == [] and s.ended == []       # nothing runs for a request with no room
    s = ScriptedSession(capacity=6)
    assert run(s, [[1, 2, 3, 4]], max_length=100) == [[5, 6]]   # clipped to the capacity


def test_stop_token_ends_a_sequence_early_and_is_not_delivered():
    s = ScriptedSession()
    seen = []
    out = run(s, [[1], [10], [20]], max_new_tokens=6, stop_ids=[13, 3],
              callback=lambda i, t: seen.append((i, t)))
    assert out == [[2], [11, 12], [21, 22, 23, 24, 25, 26]]
    # the batch shrinks as sequences stop: 3 rows, then 2 (seq 0 drew 3), then 1 ...
    assert [len(step) for step in s.steps] == [3, 3, 2, 1, 1, 1]
    assert (0, 3) not in seen and (1, 13) not in seen
    assert [t for i, t in seen if i == 2] == out[2]
    assert sorted(s.ended) == [0, 1, 2]


def test_more_requests_than_slots_run_as_consecutive_batches():
    s = ScriptedSession(max_batch=2)
    prompts = [[i] for i in range(5)]
    out = run(s, prompts, max_new_tokens=2)
    assert out == [[i + 1, i + 2] for i in range(5)]
    assert [len(step) for step in s.steps] == [2, 2, 2, 2, 1, 1]
    assert len(s.ended) == 5 and not s.live
    # sampler streams follow the request, counters its own steps
    assert argmax_sampler.calls[0] == ([0, 1], [0, 0])
    assert argmax_sampler.calls[2] == ([2, 3], [0, 0])
    assert argmax_sampler.calls[3] == ([2, 3], [1, 1])


def test_batches_respect_the_page_budget():
    requests = [Request(prompt=[1] * 10, limit=limit, stream=i)
                for i, limit in enumerate([64, 65, 128, 10, 200])]
    batches = plan_batches(requests, max_batch=8, free_tokens=4 * 64)
    assert [[r.stream for r in b] for b in batches] == [[0, 1], [2, 3], [4]]
    with pytest.raises(ValueError, match="does not fit"):
        plan_batches([Request(prompt=[1], limit=1000, stream=0)], 8, free_tokens=4 * 64)


def test_invalid_requests_are_refused_before_anything_runs():
    s = ScriptedSession()
    for prompts, kwargs in [([[]], {}), ([[1, VOCAB]], {}), ([[1] * 65], {}),
                            ([[1]], {"params": SamplingParams(top_k=0)}),
                            ([[1]], {"params": SamplingParams(top_p=0.0)}),
                            ([[1]], {"params": SamplingParams(top_p=1.5)}),
                            ([[1], [2]], {"max_length": [5]})]:
        with pytest.raises(ValueError):
            run(s, prompts, **kwargs)
    assert s.steps == [] and s.ended == [] and not s.live


def test_slots_are_returned_when_a_step_fails():
    class Failing(ScriptedSession):
        def step(self, entries, copy=True):
            if len(self.steps) == 1:
                raise RuntimeError("boom")
            return super().step(entries)
    s = Failing()
    with pytest.raises(RuntimeError, match="boom"):
        run(s, [[1], [2]], max_new_tokens=5)
    assert sorted(s.ended) == [0, 1] and not s.live


def test_sampling_params_rules():
    SamplingParams(temperature=0.0, top_k=50000).validate(100)     # min(top_k, V) counts
    assert SamplingParams(temperature=0.0, top_k=5).is_greedy(10)
    assert SamplingParams(temperature=0.7, top_k=1).is_greedy(10)
    assert SamplingParams(temperature=0.7, top_k=5).is_greedy(1)
    assert not SamplingParams(temperature=0.7, top_k=5).is_greedy(10)
    with pytest.raises(ValueError):
        SamplingParams(temperature=float("nan")).validate(10)
    with pytest.raises(ValueError, match="1024"):
        SamplingParams(temperature=1.0, top_k=2000).validate(5000)


def test_prompts_beyond_the_row_budget_run_in_portions():
    """Prompts of 5, 1, 7 and 2 tokens with room for 4 rows a step: whole prompts while they
    fit, then portions; only the step that holds a prompt's last token wants its logits, and
    the first tokens are drawn for the requests in their own order."""
    from edge_infer_amd.engine.generate import prompt_steps
    prompts = [[1, 2, 3, 4, 5], [10], [20, 21, 22, 23, 24, 25, 26], [28, 29]]
    s = ScriptedSession(max_batch=4)
    out = run(s, prompts, max_new_tokens=2, prompt_rows=4)
    assert out == [[6, 7], [11, 12], [27, 28], [30, 31]]
    prefill = s.steps[:4]
    assert [[(len(t), w) for _, t, w in step] for step in prefill] == [
        [(4, [])], [(1, [0]), (1, [0]), (2, [])], [(4, [])], [(1, [0]), (2, [1])]]
    assert [t for step in prefill for slot, t, _ in step if slot == 2] == \
        [[20, 21], [22, 23, 24, 25], [26]]
    assert all(len(t) == 1 for step in s.steps[4:] for _, t, _ in step) and len(s.steps) == 5
    # room for everything: one step, as before
    s = ScriptedSession(max_batch=4)
    assert run(s, prompts, max_new_tokens=1, prompt_rows=15) == [[6], [11], [27], [30]]
    assert len(s.steps) == 1
    requests = [Request(prompt=p, limit=99, stream=i) for i, p in enumerate(prompts)]
    assert [[(r.stream, first, count, last) for r, first, count, last in step]
            for step in prompt_steps(requests, 6)] == [
        [(0, 0, 5, True), (1, 0, 1, True)], [(2, 0, 6, False)], [(2, 6, 1, True), (3, 0, 2, True)]]
    with pytest.raises(ValueError):
        prompt_steps(requests, 0)
