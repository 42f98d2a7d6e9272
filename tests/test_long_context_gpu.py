"""Contexts of thousands of tokens at head size 128, in float32 and bfloat16, against the
plain implementation: a long prompt whole; decoding across a context bound, where the
session moves to another captured graph; a decode batch of very unequal contexts, whose key
ranges are cut into slices by the longest one; and batches of so many sequences that
attention takes its launch shapes of smaller blocks.  The q/k norm weights are raised by half, which
more than doubles the scores, so that attention is peaked: a key that is left out, read twice
or read from a foreign page then moves the logits by far more than the tolerance.  (The
rounding of bfloat16 queries and keys grows with the scores as well: with doubled weights
the bfloat16 engine is 2.1 % rms away from the plain implementation after 4,500 tokens.)"""
import pytest
import torch

import plain_qwen3 as plain
from helpers import LONG, assert_close_long as assert_close, make_long_folder, random_ids

pytestmark = pytest.mark.gpu

DTYPES = ["float32", "bfloat16"]


@pytest.fixture(scope="module")
def folder(tmp_path_factory):
    return make_long_folder(tmp_path_factory.mktemp("long"))


@pytest.fixture(scope="module")
def oracle(folder):
    cfg, weights = plain.read_folder(folder)
    cache = {}

    def logits(ids):
        key = tuple(ids)
        if key not in cache:
            cache[key] = plain.forward(weights, cfg, list(ids))
        return cache[key]
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
def test_a_prompt_of_4500_tokens_whole(models, oracle, dtype):
    import edge_infer_amd as ei
    ids = ids_of(4500, seed=1)
    session = ei.Session(models(dtype), max_tokens=4608, max_seqs=1)
    for tensor in session.cache.kv_k + session.cache.kv_v:
        tensor.fill_(float("nan"))
    places = sorted({0, 1, 63, 64, 65, 1023, 1024, 1499, 1500, 1501, 1502, 2047, 2048, 4095, 4096, 4499,
                     *range(7, 4500, 211)})
    slot = session.begin()
    logits = session.step([(slot, ids, places)])
    assert_close(dtype, logits, oracle(ids)[places], f"{dtype} 4,500 tokens whole")
    # the same sequence in portions of unequal size, two of them of two tokens (the smallest
    # item of the prompt path), one inside a page and one across the border of the first page
    # (positions 63 and 64), gives the same rows
    session.end(slot)
    slot = session.begin()
    cuts = [0, 63, 65, 1500, 1502, 4500]
    rows = []
    for begin, end in zip(cuts, cuts[1:]):
        want = [p - begin for p in places if begin <= p < end]
        rows.append(session.step([(slot, ids[begin:end], want)]))
    assert_close(dtype, torch.cat(rows), oracle(ids)[places], f"{dtype} 4,500 tokens in portions")


@pytest.mark.parametrize("dtype", DTYPES)
def test_decoding_across_a_context_bound_takes_another_graph(models, oracle, dtype):
    """1,000 prompt tokens, then 60 one by one: the sequence passes 1,024 tokens, the bound
    of the first captured step, so a second graph is captured in the middle of it; a second
    sequence of 40 tokens beside it ends before that."""
    import edge_infer_amd as ei
    from edge_infer_amd.engine.session import context_bound
    long_ids, short_ids = ids_of(4500, seed=1)[:1060], ids_of(52, seed=2)
    session = ei.Session(models(dtype), max_tokens=2048, max_seqs=2)
    assert session.graphs
    a, b = session.begin(), session.begin()
    first = session.step([(a, long_ids[:1000], [999]), (b, short_ids[:40], [39])])
    got_a, got_b = [first[0]], [first[1]]
    for t in range(60):
        entries = [(a, [long_ids[1000 + t]], [0])]
        if t < 12:
            entries.append((b, [short_ids[40 + t]], [0]))
        out = session.step(entries)
        got_a.append(out[0])
        if t < 12:
            got_b.append(out[1])
        if t == 11:
            session.end(b)
    assert_close(dtype, torch.stack(got_a), oracle(long_ids)[999:], f"{dtype} across the bound")
    assert_close(dtype, torch.stack(got_b), oracle(short_ids)[39:], f"{dtype} beside it")
    assert context_bound(1012, 5120) == 1024 and context_bound(1025, 5120) == 1536
    assert set(session._captured) == {(2, 1024), (1, 1024), (1, 1536)}
    assert session.graph_captures == 3 and session.graph_replays == 60 - 3
    # the same steps without graphs
    eager = ei.Session(models(dtype), max_tokens=2048, max_seqs=2, graphs=False)
    a = eager.begin()
    rows = [eager.step([(a, long_ids[:1000], [999])])[0]]
    rows += [eager.step([(a, [token], [0])])[0] for token in long_ids[1000:]]
    assert eager.graph_replays == 0
    assert_close(dtype, torch.stack(rows), oracle(long_ids)[999:], f"{dtype} eager")
    scale = torch.stack(rows).abs().max().item()
    bound = 1e-5 if dtype == "float32" else 3e-2
    assert (torch.stack(rows) - torch.stack(got_a)).abs().max().item() <= bound * scale


@pytest.mark.parametrize("dtype", DTYPES)
def test_a_decode_batch_of_very_unequal_contexts(models, oracle, dtype):
    """40, 1,500 and 4,300 tokens in one batch: the step's key ranges are cut into slices
    sized by the longest sequence, most of which lie beyond the short ones."""
    import edge_infer_amd as ei
    lengths = [40, 1500, 4300]
    requests = [ids_of(n + 6, seed=20 + i) for i, n in enumerate(lengths)]
    requests[2] = ids_of(4500, seed=1)[:4306]          # the oracle has these rows already
    session = ei.Session(models(dtype), max_tokens=3 * 4352, max_seqs=3, max_seq_tokens=4352)
    for tensor in session.cache.kv_k + session.cache.kv_v:
        tensor.fill_(float("nan"))
    slots = [session.begin() for _ in requests]
    out = session.step([(s, r[:n], [n - 1]) for s, r, n in zip(slots, requests, lengths)])
    got = [[row] for row in out]
    for t in range(6):
        out = session.step([(s, [r[n + t]], [0]) for s, r, n in zip(slots, requests, lengths)])
        for rows, row in zip(got, out):
            rows.append(row)
    for rows, request, n in zip(got, requests, lengths):
        assert_close(dtype, torch.stack(rows), oracle(request)[n - 1:n + 6],
                     f"{dtype} context {n} in an unequal batch")
    mixer = session.model.layers[0].mixer
    assert set(session._captured) == {(4, 4352)}
    slices, waves, heads = mixer.decode_launch(4, 4352)
    assert slices > 1, "this batch is meant to run the sliced launch shape"
    if mixer.matrix_cores:
        # few blocks: a block takes one head of the group of two
        assert waves == 16 and mixer.decode_launch(1, 300) == (1, 16, 1)


@pytest.mark.parametrize("count,waves", [(72, 8), (136, 4)])
@pytest.mark.parametrize("dtype", DTYPES)
def test_many_sequences_beyond_1024_tokens(models, oracle, dtype, count, waves):
    """72 and 136 sequences of 1,030 to 1,100 tokens: more (sequence, kv head) pairs than one
    launch of the largest blocks takes, so attention runs its shapes of 8 and of 4 waves a
    block at a context where slices matter.  Six of them are compared with the plain
    implementation, all of them with the same engine running them eight at a time (the
    16-wave shape)."""
    import edge_infer_amd as ei
    new = 3
    lengths = [1030 + (37 * i) % 71 for i in range(count)]
    requests = [ids_of(n + new, seed=100 + i) for i, n in enumerate(lengths)]
    model = models(dtype)
    mixer = model.layers[0].mixer

    def run(session, chosen):
        slots = [session.begin() for _ in chosen]
        out = session.step([(s, requests[r][:lengths[r]], [lengths[r] - 1])
                            for s, r in zip(slots, chosen)])
        rows = {r: [row] for r, row in zip(chosen, out)}
        for t in range(new):
            out = session.step([(s, [requests[r][lengths[r] + t]], [0])
                                for s, r in zip(slots, chosen)])
            for r, row in zip(chosen, out):
                rows[r].append(row)
        for s in slots:
            session.end(s)
        return {r: torch.stack(v) for r, v in rows.items()}

    wide = ei.Session(model, max_tokens=count * 1152, max_seqs=count, max_seq_tokens=1152)
    got = run(wide, list(range(count)))
    if mixer.matrix_cores:
        bucket = next(iter(wide._captured))[0]
        assert mixer.decode_launch(bucket, 1536)[1] == waves
        assert mixer.decode_launch(8, 1536)[1] == 16
    for r in (0, 1, 17, 40, 70, 71):
        n = lengths[r]
        assert_close(dtype, got[r], oracle(requests[r])[n - 1:], f"{dtype} request {r} of {count}")
    narrow = ei.Session(model, max_tokens=8 * 1152, max_seqs=8, max_seq_tokens=1152)
    bound = 1e-5 if dtype == "float32" else 3e-2
    for first in range(0, count, 8):
        chosen = list(range(first, first + 8))
        again = run(narrow, chosen)
        for r in chosen:
            scale = again[r].abs().max().item()
            assert (again[r] - got[r]).abs().max().item() <= bound * scale, f"request {r}"
