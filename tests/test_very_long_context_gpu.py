"""Contexts of tens of thousands of tokens: a prompt of 24,000 tokens through the generation
loop's own portions of 8,192 rows, decoding beyond 20,000 tokens (attention's key range in
its largest number of slices) across a context bound above 8,192 (another captured graph in
the middle of the sequence), and a batch of 100 and 20,000 tokens.  The model has one layer
of head size 128, so the plain implementation can give the logits of chosen rows alone
(keys and values of every position are cheap; a row of one layer needs no other row); its
q/k norm weights are raised so that a wrong, missing or foreign key shows.  float32 and
bfloat16, every row against the plain implementation."""
import pytest
import torch

import plain_qwen3 as plain
from helpers import LONG, assert_close_long as assert_close, make_long_folder, random_ids

pytestmark = pytest.mark.gpu

DTYPES = ["float32", "bfloat16"]
POSITIONS = 32768


@pytest.fixture(scope="module")
def folder(tmp_path_factory):
    return make_long_folder(tmp_path_factory.mktemp("very_long"), seed=6, num_hidden_layers=1,
                            max_position_embeddings=POSITIONS)


@pytest.fixture(scope="module")
def oracle(folder):
    cfg, weights = plain.read_folder(folder)

    def logits(ids, rows):
        return plain.forward(weights, cfg, list(ids), rows=list(rows))
    return logits


@pytest.fixture(scope="module")
def models(folder):
    import edge_infer_amd as ei
    cache = {}

    def get(dtype):
        if dtype not in cache:
            cache[dtype] = ei.load_model(folder, dtype=dtype)
        return cache[dtype]
    return get


def ids_of(count, seed):
    return random_ids(LONG["vocab_size"], count, seed)


@pytest.mark.parametrize("dtype", DTYPES)
def test_a_prompt_of_24000_tokens_in_the_loops_portions(models, oracle, dtype):
    import edge_infer_amd as ei
    from edge_infer_amd.engine.generate import PROMPT_ROWS, Request, _prefill, prompt_steps
    ids = ids_of(24000, seed=1)
    session = ei.Session(models(dtype), max_tokens=24064, max_seqs=1)
    for tensor in session.cache.kv_k + session.cache.kv_v:
        tensor.fill_(float("nan"))
    request = Request(prompt=ids, limit=24010, stream=0)
    assert PROMPT_ROWS == 8192
    assert [[(first, count) for _, first, count, _ in step]
            for step in prompt_steps([request], PROMPT_ROWS)] == \
        [[(0, 8192)], [(8192, 8192)], [(16384, 7616)]]
    request.slot = session.begin()
    last = _prefill(session, [request], PROMPT_ROWS)
    assert_close(dtype, last, oracle(ids, [23999]), f"{dtype} the last row of 24,000")
    session.end(request.slot)
    # the same portions with rows wanted inside them: the ends of portions and pages, the
    # first rows of the next ones, rows deep inside
    places = sorted({0, 63, 64, 4095, 4096, 8190, 8191, 8192, 8193, 12287, 12288, 16383, 16384,
                     16385, 20479, 20480, 23998, 23999, *range(11, 24000, 1733)})
    slot = session.begin()
    rows = []
    for first in range(0, 24000, PROMPT_ROWS):
        stop = min(24000, first + PROMPT_ROWS)
        rows.append(session.step([(slot, ids[first:stop],
                                   [p - first for p in places if first <= p < stop])]))
    assert_close(dtype, torch.cat(rows), oracle(ids, places), f"{dtype} rows of 24,000 in portions")
    # the whole loop over the same prompt, greedy: its first token is the last row's best one
    session.end(slot)
    tokens = session.generate_batch([ids], max_new_tokens=3, temperature=0.0, stop_ids=())[0]
    expected = oracle(ids, [23999])[0]
    if dtype == "float32":
        assert tokens[0] == int(expected.argmax())
    else:
        assert expected.max() - expected[tokens[0]] <= 0.03 * expected.abs().max()
    follow = oracle(ids + tokens[:2], [24000, 24001])
    for row, token in zip(follow, tokens[1:]):
        assert row.max() - row[token] <= (1e-4 if dtype == "float32" else 0.03) * row.abs().max()


@pytest.mark.parametrize("dtype", DTYPES)
def test_decoding_beyond_20000_tokens_across_a_context_bound(models, oracle, dtype):
    """24,560 prompt tokens, then 40 one by one: the sequence passes 24,576, where the
    session moves from the graph of that bound to the one of the next, 32,768; the key range
    is cut into the most slices attention has."""
    import edge_infer_amd as ei
    from edge_infer_amd.engine.session import context_bound
    ids = ids_of(24600, seed=2)
    session = ei.Session(models(dtype), max_tokens=32768, max_seqs=1)
    for tensor in session.cache.kv_k + session.cache.kv_v:
        tensor.fill_(float("nan"))
    slot = session.begin()
    rows = [session.step([(slot, ids[:24560], [24559])])]
    rows += [session.step([(slot, [token], [0])]) for token in ids[24560:]]
    assert_close(dtype, torch.cat(rows), oracle(ids, range(24559, 24600)),
                 f"{dtype} decoding at 24,600 tokens")
    assert context_bound(24570, POSITIONS) == 24576 and context_bound(24577, POSITIONS) == 32768
    assert set(session._captured) == {(1, 24576), (1, 32768)}
    assert session.graph_captures == 2 and session.graph_replays == 38
    mixer = session.model.layers[0].mixer
    from edge_infer_amd.parts.attention import MAX_SLICES
    assert mixer.decode_launch(1, 24576)[0] == MAX_SLICES == 32
    # the same without graphs: launch shapes follow the true length at every step
    eager = ei.Session(models(dtype), max_tokens=24640, max_seqs=1, graphs=False)
    slot = eager.begin()
    eager.step([(slot, ids[:24560], [])])
    again = torch.cat([eager.step([(slot, [token], [0])]) for token in ids[24560:24572]])
    assert_close(dtype, again, oracle(ids, range(24560, 24572)), f"{dtype} eager at 24,570 tokens")


@pytest.mark.parametrize("dtype", DTYPES)
def test_a_batch_of_100_and_20000_tokens(models, oracle, dtype):
    """Both prompts in one step (20,100 packed rows), then eight tokens each in one decode
    batch whose slices are sized by the long sequence: all but the first lie beyond the short
    one."""
    import edge_infer_amd as ei
    lengths = [100, 20000]
    requests = [ids_of(n + 8, seed=30 + i) for i, n in enumerate(lengths)]
    session = ei.Session(models(dtype), max_tokens=20480 + 128, max_seqs=2)
    for tensor in session.cache.kv_k + session.cache.kv_v:
        tensor.fill_(float("nan"))
    slots = [session.begin(), session.begin()]
    out = session.step([(s, r[:n], [n - 1]) for s, r, n in zip(slots, requests, lengths)])
    got = [[row] for row in out]
    for t in range(8):
        out = session.step([(s, [r[n + t]], [0]) for s, r, n in zip(slots, requests, lengths)])
        for rows, row in zip(got, out):
            rows.append(row)
    for rows, request, n in zip(got, requests, lengths):
        assert_close(dtype, torch.stack(rows), oracle(request, range(n - 1, n + 8)),
                     f"{dtype} context {n} beside the other")
    assert session.graph_replays == 7


@pytest.mark.parametrize("dtype", DTYPES)
def test_eight_like_prompts_take_paired_work_items(models, oracle, dtype, monkeypatch):
    """Eight prompts of 2,048 tokens in one step: enough work items of like prompts for the
    matrix-core prefill kernel to run one wave a key range (`key_ways` 1) and to give every
    block a long item and a short one (`pair_items`), which a single prompt never reaches."""
    import edge_infer_amd as ei
    from edge_infer_amd.csrc import lib
    seen = []
    launch = lib.attention_prefill_mfma

    def spy(*args, **kwargs):
        seen.append((kwargs["key_ways"], kwargs["pair_items"], args[6]))
        return launch(*args, **kwargs)
    monkeypatch.setattr(lib, "attention_prefill_mfma", spy)
    prompts = [ids_of(2048, seed=50 + i) for i in range(8)]
    session = ei.Session(models(dtype), max_tokens=8 * 2048, max_seqs=8)
    for tensor in session.cache.kv_k + session.cache.kv_v:
        tensor.fill_(float("nan"))
    slots = [session.begin() for _ in prompts]
    places = [0, 1, 63, 64, 127, 128, 1000, 1023, 1024, 1919, 1920, 2046, 2047]
    logits = session.step([(slot, prompt, places) for slot, prompt in zip(slots, prompts)])
    for index, prompt in enumerate(prompts):
        assert_close(dtype, logits[index * len(places):(index + 1) * len(places)],
                     oracle(prompt, places), f"{dtype} prompt {index} of eight")
    mixer = session.model.layers[0].mixer
    if mixer.matrix_cores:
        items = 8 * 2048 // mixer.positions_per_item(1)
        assert mixer.prefill_key_ways([2048] * 8) == 1 and seen == [(1, True, items)]
        assert items * mixer.spec.n_kv_heads >= 2 * mixer.compute_units     # the kernel pairs them
    else:
        assert not seen
