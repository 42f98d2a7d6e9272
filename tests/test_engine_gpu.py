"""The engine against the plain implementation, in float32 and in bfloat16: requests
alone and whole, their last 32 tokens one by one, batches of unequal lengths with slot
reuse, long decoding, first tokens, generation through the entry point."""
import pytest
import torch

import plain_qwen3 as plain
from helpers import assert_close, make_folder, random_ids, tiny_config

pytestmark = pytest.mark.gpu

DTYPES = ["float32", "bfloat16"]
NAMES = ["A", "B"]


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    root = tmp_path_factory.mktemp("models")
    return {name: make_folder(name, root) for name in NAMES}


@pytest.fixture(scope="module")
def oracle(folders):
    return {name: plain.read_folder(folders[name]) for name in NAMES}


@pytest.fixture(scope="module")
def models(folders):
    import edge_infer_amd as ei
    cache = {}

    def get(name, dtype):
        if (name, dtype) not in cache:
            cache[(name, dtype)] = ei.load_model(folders[name], dtype=dtype)
        return cache[(name, dtype)]
    return get


def requests_for(name, lengths, seed=11):
    vocab = tiny_config(name).vocab_size
    return [random_ids(vocab, n, seed + i) for i, n in enumerate(lengths)]


LENGTHS = {"A": [100, 33, 65, 120], "B": [40, 33, 200, 64, 129]}


@pytest.fixture(scope="module")
def references(oracle):
    out = {}
    for name in NAMES:
        cfg, w = oracle[name]
        out[name] = [plain.forward(w, cfg, ids) for ids in requests_for(name, LENGTHS[name])]
    return out


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", NAMES)
def test_each_request_alone_and_whole(models, references, name, dtype):
    import edge_infer_amd as ei
    session = ei.Session(models(name, dtype), max_tokens=256)
    for ids, ref in zip(requests_for(name, LENGTHS[name]), references[name]):
        slot = session.begin()
        logits = session.step([(slot, ids, list(range(len(ids))))])
        assert_close(dtype, logits, ref, f"{name} {dtype} whole {len(ids)}")
        if dtype == "float32":
            assert torch.equal(logits.argmax(-1).cpu(), ref.argmax(-1))
        session.end(slot)
    session.cache.check()


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", NAMES)
def test_last_32_tokens_one_by_one(models, references, name, dtype):
    import edge_infer_amd as ei
    session = ei.Session(models(name, dtype), max_tokens=256)
    for ids, ref in zip(requests_for(name, LENGTHS[name]), references[name]):
        cut = len(ids) - 32
        slot = session.begin()
        rows = [session.step([(slot, ids[:cut], [cut - 1])])]
        for t in range(cut, len(ids)):
            rows.append(session.step([(slot, [ids[t]], [0])]).clone())
        assert session.length(slot) == len(ids)
        assert_close(dtype, torch.cat(rows), ref[cut - 1:], f"{name} {dtype} tail {len(ids)}")
        session.end(slot)


def run_batches(session, requests, batches, tail=32):
    """Each batch: prefixes in one step, then one token each; shorter requests end
    earlier and their slots go back at once.  Returns per request the logits at the last
    prefix row and at every later token."""
    got = {}
    for batch in batches:
        slots = {r: session.begin() for r in batch}
        cuts = {r: max(1, len(requests[r]) - tail) for r in batch}
        logits = session.step([(slots[r], requests[r][:cuts[r]], [cuts[r] - 1]) for r in batch])
        for i, r in enumerate(batch):
            got[r] = [logits[i].clone()]
        at = dict(cuts)
        live = [r for r in batch if at[r] < len(requests[r])]
        for r in batch:
            if r not in live:
                session.end(slots[r])
        while live:
            logits = session.step([(slots[r], [requests[r][at[r]]], [0]) for r in live])
            for i, r in enumerate(live):
                got[r].append(logits[i].clone())
                at[r] += 1
            for r in [r for r in live if at[r] >= len(requests[r])]:
                session.end(slots[r])
            live = [r for r in live if at[r] < len(requests[r])]
        session.cache.check()
    return {r: torch.stack(rows) for r, rows in got.items()}


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", NAMES)
def test_batches_of_unequal_lengths_one_after_another(models, references, name, dtype):
    """Slots and pages are used again by the second and third batch; the cache is filled
    with NaN first so that a read of a stale or foreign position shows."""
    import edge_infer_amd as ei
    requests = requests_for(name, LENGTHS[name])
    n = len(requests)
    session = ei.Session(models(name, dtype), max_tokens=7 * 64, max_seqs=3)
    for tensor in session.cache.kv_k + session.cache.kv_v:
        tensor.fill_(float("nan"))
    order = list(range(n))
    batches = [order[:3], order[3:] + [0], [2, 1]]
    for batch_set in (batches[:2], batches[2:]):
        got = run_batches(session, requests, batch_set)
        for r, rows in got.items():
            cut = max(1, len(requests[r]) - 32)
            assert_close(dtype, rows, references[name][r][cut - 1:],
                         f"{name} {dtype} batched request {r}")
    assert session.cache.slots.n_free == 3
    assert all(pool.n_free == pool.n_pages for pool in session.cache.kv_pools)


@pytest.mark.parametrize("dtype", DTYPES)
def test_random_schedules_against_the_plain_implementation(models, oracle, dtype):
    """Seeded random traffic on one session: requests of 1 to 120 tokens in batches of 1 to 4
    that follow each other on 4 slots and a page budget that is just enough, with tails of
    random lengths decoded token by token; every returned row against the plain logits."""
    import random
    import edge_infer_amd as ei
    name = "B"
    cfg, w = oracle[name]
    rng = random.Random(2024)
    session = ei.Session(models(name, dtype), max_tokens=4 * 128, max_seqs=4)
    for tensor in session.cache.kv_k + session.cache.kv_v:
        tensor.fill_(float("nan"))
    cache = {}
    for scenario in range(6):
        n = rng.randint(1, 4)
        lengths = [rng.randint(1, 120) for _ in range(n)]
        requests = [random_ids(cfg["vocab_size"], length, 1000 * scenario + i)
                    for i, length in enumerate(lengths)]
        tail = rng.choice([0, 1, 7, 40])
        got = run_batches(session, requests, [list(range(n))], tail=tail)
        for r, rows in got.items():
            key = tuple(requests[r])
            if key not in cache:
                cache[key] = plain.forward(w, cfg, requests[r])
            cut = max(1, len(requests[r]) - tail)
            assert_close(dtype, rows, cache[key][cut - 1:],
                         f"{dtype} scenario {scenario} request {r} of lengths {lengths} tail {tail}")
        assert session.cache.slots.n_free == 4
    assert all(pool.n_free == pool.n_pages for pool in session.cache.kv_pools)


@pytest.mark.parametrize("dtype", DTYPES)
def test_batch_composition_changes_nothing(models, dtype):
    """The same request alone and inside two different batches: in float32 the rows are
    bit-identical (every kernel reduces in an order that ignores the neighbours)."""
    import edge_infer_amd as ei
    name = "B"
    requests = requests_for(name, [70, 5, 64, 131], seed=31)
    session = ei.Session(models(name, dtype), max_tokens=1024)
    alone = run_batches(session, requests, [[0]])[0]
    mixed = run_batches(session, requests, [[1, 0, 3, 2]])[0]
    other = run_batches(session, requests, [[3, 0]])[0]
    if dtype == "float32":
        assert torch.equal(alone, mixed) and torch.equal(alone, other)
    else:
        scale = alone.abs().max().item()
        assert (alone - mixed).abs().max().item() <= 0.02 * scale
        assert (alone - other).abs().max().item() <= 0.02 * scale


@pytest.mark.parametrize("dtype", DTYPES)
def test_a_batch_wider_than_64_sequences(models, oracle, dtype):
    """70 short requests of 3 to 12 tokens start together and end one after another, so the
    decode steps run with 70, then fewer and fewer rows: past 64 rows the few-rows product
    works in groups of 64 rows (bfloat16), and every batch bucket on the way down is used."""
    import edge_infer_amd as ei
    name = "A"
    cfg, w = oracle[name]
    lengths = [3 + (7 * i) % 10 for i in range(70)]
    requests = requests_for(name, lengths, seed=501)
    session = ei.Session(models(name, dtype), max_tokens=70 * 64, max_seqs=70)
    got = run_batches(session, requests, [list(range(70))], tail=8)
    for r in (0, 1, 17, 63, 64, 65, 69):
        ref = plain.forward(w, cfg, requests[r])
        cut = max(1, len(requests[r]) - 8)
        assert_close(dtype, got[r], ref[cut - 1:], f"{dtype} request {r} of a batch of 70")
    assert session.cache.slots.n_free == 70


@pytest.mark.parametrize("dtype", DTYPES)
def test_a_decode_batch_beyond_the_few_rows_product(models, oracle, dtype):
    """260 sequences decode together: more rows than the weight-streaming product takes, so
    the bfloat16 step multiplies through the library, runs eagerly and prepares queries and
    keys with the kernel of their own; as sequences end it comes back under 256 rows and
    to the graphs."""
    import edge_infer_amd as ei
    name = "B"
    cfg, w = oracle[name]
    lengths = [4 + (5 * i) % 7 for i in range(260)]
    requests = requests_for(name, lengths, seed=901)
    session = ei.Session(models(name, dtype), max_tokens=260 * 64, max_seqs=260)
    got = run_batches(session, requests, [list(range(260))], tail=6)
    for r in (0, 1, 100, 255, 256, 259):
        ref = plain.forward(w, cfg, requests[r])
        cut = max(1, len(requests[r]) - 6)
        assert_close(dtype, got[r], ref[cut - 1:], f"{dtype} request {r} of a batch of 260")
    assert session.cache.slots.n_free == 260


@pytest.mark.parametrize("dtype", DTYPES)
def test_long_decoding_and_first_tokens(models, oracle, dtype):
    """A prompt of one token, then 230 tokens one by one across three page boundaries."""
    import edge_infer_amd as ei
    name = "B"
    cfg, w = oracle[name]
    ids = random_ids(cfg["vocab_size"], 231, 77)
    ref = plain.forward(w, cfg, ids)
    session = ei.Session(models(name, dtype), max_tokens=256)
    slot = session.begin()
    rows = [session.step([(slot, ids[:1], [0])]).clone()]
    for t in range(1, len(ids)):
        rows.append(session.step([(slot, [ids[t]], [0])]).clone())
    got = torch.cat(rows)
    assert_close(dtype, got[:4], ref[:4], f"{dtype} first tokens")
    assert_close(dtype, got, ref, f"{dtype} long decode")
    # chunks of odd sizes give the same rows again
    session.end(slot)
    slot = session.begin()
    rows, at = [], 0
    for size in (3, 61, 1, 64, 70, 32):
        rows.append(session.step([(slot, ids[at:at + size], list(range(size)))]).clone())
        at += size
    assert_close(dtype, torch.cat(rows), ref[:at], f"{dtype} chunked")


def test_refused_steps_change_nothing(models):
    import edge_infer_amd as ei
    from edge_infer_amd.cache import CacheFull
    session = ei.Session(models("A", "float32"), max_tokens=128, max_seqs=2)
    slot = session.begin()
    session.step([(slot, [1, 2, 3], [2])])
    before = session.cache.kv_k[0].clone()
    for entries in ([(slot, [256], [0])], [(slot, [-1], [0])], [(slot, [], [])],
                    [(slot, [1], [1])], [(5, [1], [0])], [(slot, [1], [0]), (slot, [2], [0])],
                    [(slot, [1.0], [0])], [(slot, [True], [0])]):
        with pytest.raises(ValueError):
            session.step(entries)
    import numpy as np
    again = session.step([(slot, [np.int64(7), np.int32(9)], [1])])     # integers of any kind
    assert again.shape == (1, 256) and session.length(slot) == 5
    session.end(slot)
    slot = session.begin()
    session.step([(slot, [1, 2, 3], [2])])
    before = session.cache.kv_k[0].clone()
    with pytest.raises(CacheFull):
        session.step([(slot, [1] * 126, [])])          # 3 + 126 > 128 positions of the model
    other = session.begin()
    with pytest.raises(CacheFull):
        session.step([(other, [1] * 100, [])])          # no second page pair free
    assert session.length(slot) == 3 and session.length(other) == 0
    assert torch.equal(before.view(torch.int32), session.cache.kv_k[0].view(torch.int32))
    with pytest.raises(CacheFull):
        session.begin()
    session.end(other)
    with pytest.raises(RuntimeError):
        session.end(other)
    session.cache.check()


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", NAMES)
def test_greedy_generation_through_the_entry_point(folders, oracle, name, dtype):
    """The workload of the tiny configurations: a batch of unequal prompts, then
    greedy decoding, against the plain implementation that recomputes whole sequences."""
    from edge_infer_amd.api import Model
    cfg, w = oracle[name]
    lengths, new = ([5, 11, 17], 8) if name == "A" else ([1, 7, 30, 64], 12)
    prompts = requests_for(name, lengths, seed=91)
    model = Model.from_pretrained(folders[name], "qwen3_fp32" if dtype == "float32" else "qwen3_bf16")
    session = model.new_session(capacity=128, max_batch=len(prompts))
    seen = []
    got = session.generate_batch(prompts, max_new_tokens=new, temperature=0.0, stop_ids=(),
                                 callback=lambda i, t: seen.append((i, t)))
    for i, prompt in enumerate(prompts):
        expected = plain.generate(w, cfg, prompt, max_length=len(prompt) + new, stop_ids=set())
        if dtype == "float32":
            assert got[i] == expected, f"request {i}"
        else:
            # bfloat16 may leave the greedy path where two logits are within its error;
            # up to there the tokens agree, and the step that differs is a near tie
            agree = 0
            while agree < len(expected) and got[i][agree] == expected[agree]:
                agree += 1
            if agree < len(expected):
                logits = plain.forward(w, cfg, prompt + expected[:agree])[-1]
                gap = (logits[expected[agree]] - logits[got[i][agree]]).item()
                assert 0 <= gap <= 0.03 * logits.abs().max().item(), f"request {i} step {agree}"
        assert [t for j, t in seen if j == i] == got[i]
    # the single-request call of the reference's API: max_length counts the prompt
    single = session.generate(prompts[1], max_length=len(prompts[1]) + 4, top_k=1)
    first4 = plain.generate(w, cfg, prompts[1], max_length=len(prompts[1]) + 4)
    if dtype == "float32":
        assert single == first4
    else:
        # alone, the request runs other launch shapes than in the batch; it may leave the
        # plain implementation's greedy path only at a near tie, like the batch above
        agree = 0
        while agree < min(len(single), len(first4)) and single[agree] == first4[agree]:
            agree += 1
        if agree < len(first4):
            assert agree < len(single), "the request ended early"
            logits = plain.forward(w, cfg, prompts[1] + first4[:agree])[-1]
            gap = (logits[first4[agree]] - logits[single[agree]]).item()
            assert 0 <= gap <= 0.03 * logits.abs().max().item(), f"alone, step {agree}"
    assert session.generate(prompts[1], max_length=len(prompts[1])) == []
    # the end-of-sequence token ends a request and is not delivered
    if dtype == "float32":
        stop = got[0][2]
        cut = session.generate_batch([prompts[0]], max_new_tokens=new, temperature=0.0,
                                     stop_ids=(stop,))[0]
        assert cut == got[0][:got[0].index(stop)]


def test_procedural_interface_generates_like_a_session(folders, oracle):
    """init_model / generate_text_stream (bindings/python/model_bridge.cpp:171-193): the
    implicit session gives the tokens of an explicit one; a failed init keeps the old model;
    a callback that calls back in is refused."""
    from edge_infer_amd import api
    cfg, w = oracle["A"]
    prompt = requests_for("A", [9], seed=77)[0]
    config, weights, model_type = api.load_checkpoint(folders["A"], "qwen3_fp32")
    assert api.init_model(config, weights, model_type) is True
    got = []
    api.generate_text_stream(prompt, got.append, max_length=len(prompt) + 6, top_k=1)
    expected = plain.generate(w, cfg, prompt, max_length=len(prompt) + 6)
    assert got == expected
    assert api.init_model({"architectures": ["NoSuchModel"]}, {}, "qwen3_fp32") is False
    again = []
    api.generate_text_stream(prompt, again.append, max_length=len(prompt) + 6, top_k=1)
    assert again == got

    def nested(token):
        with pytest.raises(RuntimeError, match="busy"):
            api.generate_text_stream(prompt, lambda t: None, max_length=len(prompt) + 1)
    api.generate_text_stream(prompt, nested, max_length=len(prompt) + 2, top_k=1)
    session = api._compat["session"]
    assert session.speculative is False and session.capacity == min(4096, cfg["max_position_embeddings"])
    api._compat["model"] = api._compat["session"] = None


def test_a_session_refuses_a_second_operation_while_one_runs(models):
    """bindings/python/include/python_callback.hpp:16-26: a callback that generates or resets
    on its own session is refused; the running generation goes on and ends cleanly."""
    import edge_infer_amd as ei
    session = ei.Session(models("A", "float32"), max_tokens=256, max_seqs=2)
    prompt = requests_for("A", [6], seed=3)[0]
    refused = []

    def callback(index, token):
        for action in (lambda: session.generate(prompt, max_length=8), session.reset):
            with pytest.raises(RuntimeError, match="busy"):
                action()
            refused.append(token)
    out = session.generate_batch([prompt], max_new_tokens=3, temperature=0.0, stop_ids=(),
                                 callback=callback)[0]
    assert len(out) == 3 and len(refused) == 6
    assert session.generate_batch([prompt], max_new_tokens=3, temperature=0.0, stop_ids=())[0] == out
    session.reset()
    assert session.cache.slots.n_free == 2


def test_seeded_sampling_is_the_same_alone_and_in_a_batch(folders, oracle):
    """Configuration B's workload: temperature 0.8 with a seeded sampler.  Every drawn
    token equals the plain sampler's draw from the plain logits of the same prefix."""
    from edge_infer_amd.api import Model
    cfg, w = oracle["B"]
    prompts = requests_for("B", [1, 7, 30, 64], seed=17)
    model = Model.from_pretrained(folders["B"], "qwen3_fp32")
    session = model.new_session(capacity=128, max_batch=4, seed=2024)
    kwargs = dict(max_new_tokens=12, temperature=0.8, top_p=0.95, top_k=40, stop_ids=())
    together = session.generate_batch(prompts, first_stream=0, **kwargs)
    for i, prompt in enumerate(prompts):
        alone = session.generate_batch([prompt], first_stream=i, **kwargs)[0]
        assert alone == together[i]
        ids = list(prompt)
        for step, token in enumerate(together[i]):
            logits = plain.forward(w, cfg, ids)[-1].float().numpy()
            assert token == plain.sample(logits, 0.8, 0.95, 40, plain.uniform(2024, i, step)), \
                f"request {i} step {step}"
            ids.append(token)
    assert len({tuple(t) for t in together}) == 4
    again = session.generate_batch(prompts, first_stream=0, seed=7, **kwargs)
    assert again != together


@pytest.mark.parametrize("fused", [True, False])
@pytest.mark.parametrize("dtype", DTYPES)
def test_head_size_64_with_groups_of_eight(tmp_path, dtype, fused, monkeypatch):
    """A third shape, for the matrix-core attention at head size 64: 16 query heads on 2 kv
    heads (decode blocks of 16 waves then take a group in two blocks), an intermediate size
    that is no multiple of 16 (gate and up stay halves), an odd vocabulary; whole prompts of
    unequal lengths, then token by token.  Decode with the attention kernel making its own
    queries and keys, and with the separate kernel for that (which batches beyond 256 rows
    take)."""
    import edge_infer_amd as ei
    from edge_infer_amd.parts import attention
    monkeypatch.setattr(attention, "FUSED_DECODE", fused)
    cfg = ei.Qwen3Config(vocab_size=777, hidden_size=192, num_hidden_layers=2,
                         num_attention_heads=16, num_key_value_heads=2, head_dim=64,
                         intermediate_size=296, max_position_embeddings=512, bos_token_id=0,
                         eos_token_id=776, rms_norm_eps=1e-5, rope_theta=50000.0,
                         tie_word_embeddings=True)
    folder = ei.write_model_folder(tmp_path / "d64", cfg, seed=8)
    pcfg, pw = plain.read_folder(folder)
    prompts = [random_ids(777, n, 40 + n) for n in (150, 31, 260)]
    refs = [plain.forward(pw, pcfg, ids) for ids in prompts]
    session = ei.Session(ei.load_model(folder, dtype=dtype), max_tokens=1024, max_seqs=3)
    slots = [session.begin() for _ in prompts]
    cuts = [len(p) - 12 for p in prompts]
    logits = session.step([(s, p[:c], [c - 1]) for s, p, c in zip(slots, prompts, cuts)])
    rows = [[logits[i]] for i in range(3)]
    for t in range(12):
        out = session.step([(s, [p[c + t]], [0]) for s, p, c in zip(slots, prompts, cuts)])
        for i in range(3):
            rows[i].append(out[i])
    for i in range(3):
        assert_close(dtype, torch.stack(rows[i]), refs[i][cuts[i] - 1:], f"d64 {dtype} request {i}")
    if dtype == "bfloat16":
        assert session.graph_replays > 0


@pytest.mark.parametrize("dtype", DTYPES)
def test_widths_that_are_no_multiple_of_eight(tmp_path, dtype):
    """Hidden size 100, intermediate size 52, vocabulary 99: the few-rows product needs a K
    that is a multiple of 8 and is not taken here (the library multiplies, decode is not
    captured); the row-wise kernels take their scalar forms.  Results are the same."""
    import edge_infer_amd as ei
    cfg = ei.Qwen3Config(vocab_size=99, hidden_size=100, num_hidden_layers=2,
                         num_attention_heads=3, num_key_value_heads=1, head_dim=16,
                         intermediate_size=52, max_position_embeddings=128, bos_token_id=0,
                         eos_token_id=98, rms_norm_eps=1e-6, rope_theta=10000.0,
                         tie_word_embeddings=False)
    folder = ei.write_model_folder(tmp_path / "odd", cfg, seed=12)
    pcfg, pw = plain.read_folder(folder)
    prompts = [random_ids(99, n, 60 + n) for n in (70, 9)]
    refs = [plain.forward(pw, pcfg, ids) for ids in prompts]
    session = ei.Session(ei.load_model(folder, dtype=dtype), max_tokens=256, max_seqs=2)
    slots = [session.begin() for _ in prompts]
    cuts = [len(p) - 5 for p in prompts]
    logits = session.step([(s, p[:c], [c - 1]) for s, p, c in zip(slots, prompts, cuts)])
    rows = [[logits[i]] for i in range(2)]
    for t in range(5):
        out = session.step([(s, [p[c + t]], [0]) for s, p, c in zip(slots, prompts, cuts)])
        for i in range(2):
            rows[i].append(out[i])
    for i in range(2):
        assert_close(dtype, torch.stack(rows[i]), refs[i][cuts[i] - 1:], f"odd {dtype} request {i}")


@pytest.mark.parametrize("dtype", DTYPES)
def test_one_layer_of_the_8b_shape(tmp_path, dtype):
    """Layer sizes of Qwen3-8B (hidden 4096, 32 heads, 8 kv heads, head_dim 128,
    intermediate 12288) with one layer and a small vocabulary: the kernels that the big
    model uses (matrix-core attention, few-rows and library products at K = 4096 and
    12288) against the plain implementation, whole and token by token, two sequences.  The
    370 prompt rows of the first step are beyond the few-rows product and go to the library."""
    import edge_infer_amd as ei
    cfg = ei.Qwen3Config(vocab_size=1000, hidden_size=4096, num_hidden_layers=1,
                         num_attention_heads=32, num_key_value_heads=8, head_dim=128,
                         intermediate_size=12288, max_position_embeddings=512, bos_token_id=0,
                         eos_token_id=999, rms_norm_eps=1e-6, rope_theta=1e6,
                         tie_word_embeddings=False)
    folder = ei.write_model_folder(tmp_path / "layer8b", cfg, seed=2)
    pcfg, pw = plain.read_folder(folder)
    a, b = random_ids(1000, 330, 5), random_ids(1000, 70, 6)
    ref_a, ref_b = plain.forward(pw, pcfg, a), plain.forward(pw, pcfg, b)
    model = ei.load_model(folder, dtype=dtype)
    session = ei.Session(model, max_tokens=1024, max_seqs=2)
    sa, sb = session.begin(), session.begin()
    logits = session.step([(sa, a[:310], list(range(310))), (sb, b[:60], list(range(60)))])
    assert_close(dtype, logits[:310], ref_a[:310], f"8B-shape layer {dtype} prefill a")
    assert_close(dtype, logits[310:], ref_b[:60], f"8B-shape layer {dtype} prefill b")
    rows_a, rows_b = [], []
    for t in range(20):
        entries = [(sa, [a[310 + t]], [0])]
        if t < 10:
            entries.append((sb, [b[60 + t]], [0]))
        out = session.step(entries)
        rows_a.append(out[0])
        if t < 10:
            rows_b.append(out[1])
    assert_close(dtype, torch.stack(rows_a), ref_a[310:], f"8B-shape layer {dtype} decode a")
    assert_close(dtype, torch.stack(rows_b), ref_b[60:], f"8B-shape layer {dtype} decode b")
    assert session.graph_replays > 0


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("which", ["all", "some"])
def test_projection_biases(tmp_path, dtype, which):
    """The optional biases of the projections and of the head
    (runtime/include/models/qwen3_model.hpp:371-403), made eight times as large as they are
    drawn so that a dropped or misplaced one shows.  "all": an intermediate size in whole
    strips of 16 (gate and up rows interleave, and so must their biases).  "some": no v,
    up or down bias (absent ones count as zero), an intermediate size that keeps gate and up
    as halves, a tied head with a bias.  A first step of 347 rows goes to the library's
    product in bfloat16, a second batch of few rows to the weight-streaming kernel; then
    token by token."""
    import edge_infer_amd as ei
    from safetensors.torch import load_file, save_file
    cfg = ei.Qwen3Config(vocab_size=333, hidden_size=128, num_hidden_layers=2,
                         num_attention_heads=4, num_key_value_heads=2, head_dim=32,
                         intermediate_size=208 if which == "all" else 200,
                         max_position_embeddings=512, bos_token_id=0, eos_token_id=332,
                         rms_norm_eps=1e-6, rope_theta=10000.0,
                         tie_word_embeddings=which == "some")
    folder = ei.write_model_folder(tmp_path / f"biased_{which}", cfg, seed=21, biases=True)
    path = str(folder / "model.safetensors")
    tensors = {}
    for name, tensor in load_file(path).items():
        if name.endswith(".bias"):
            if which == "some" and any(part in name for part in ("v_proj", "up_proj", "down_proj")):
                continue
            tensor = (tensor.float() * 8).to(tensor.dtype)
        tensors[name] = tensor
    assert sum(name.endswith(".bias") for name in tensors) == (15 if which == "all" else 9)
    save_file(tensors, path, metadata={"format": "pt"})
    pcfg, pw = plain.read_folder(folder)
    prompts = [random_ids(333, n, 80 + n) for n in (300, 40, 7, 90, 12)]
    refs = [plain.forward(pw, pcfg, ids) for ids in prompts]
    # the biases matter: without them the logits are far off
    bare = {name: t for name, t in pw.items() if not name.endswith(".bias")}
    assert (plain.forward(bare, pcfg, prompts[2]) - refs[2]).abs().max() > 0.1 * refs[2].abs().max()
    session = ei.Session(ei.load_model(folder, dtype=dtype), max_tokens=1024, max_seqs=3)
    for batch in ([0, 1, 2], [3, 4]):
        slots = [session.begin() for _ in batch]
        cuts = [len(prompts[i]) - 5 for i in batch]
        logits = session.step([(s, prompts[i][:c], [0, c - 1])
                               for s, i, c in zip(slots, batch, cuts)])
        rows = {i: [logits[2 * j + 1]] for j, i in enumerate(batch)}
        for j, (i, c) in enumerate(zip(batch, cuts)):
            assert_close(dtype, logits[2 * j][None], refs[i][:1], f"biases {which} first row {i}")
        for t in range(5):
            out = session.step([(s, [prompts[i][c + t]], [0])
                                for s, i, c in zip(slots, batch, cuts)])
            for j, i in enumerate(batch):
                rows[i].append(out[j])
        for i, c in zip(batch, cuts):
            assert_close(dtype, torch.stack(rows[i]), refs[i][c - 1:], f"biases {which} {dtype} {i}")
        for s in slots:
            session.end(s)
    if dtype == "bfloat16":
        assert session.graph_replays > 0


@pytest.mark.parametrize("dtype", DTYPES)
def test_planned_workspace_gives_the_same_logits_in_less_storage(models, references, dtype):
    """The first step of a shape runs on one buffer per name and records lifetimes; the
    next step of that shape runs in the planned arena, where dead intermediates share
    storage: the same logits bit for bit, fewer bytes, and the plan holds no two live values
    in one place (its constructor checks that)."""
    import edge_infer_amd as ei
    session = ei.Session(models("B", dtype), max_tokens=1024, max_seqs=4, graphs=False)
    prompts = requests_for("B", LENGTHS["B"])[:3]
    results = []
    for _ in range(3):
        slots = [session.begin() for _ in prompts]
        logits = session.step([(s, p, [0, len(p) - 1]) for s, p in zip(slots, prompts)])
        tokens = [[1], [2], [3]]
        decoded = session.step([(s, t, [0]) for s, t in zip(slots, tokens)])
        results.append((logits, decoded))
        for s in slots:
            session.end(s)
    for logits, decoded in results[1:]:
        assert torch.equal(logits, results[0][0]) and torch.equal(decoded, results[0][1])
    for i, p in enumerate(prompts):
        assert_close(dtype, results[2][0][2 * i + 1][None], references["B"][i][-1:], "planned")
    plans = list(session.workspace._plans.values())
    assert len(plans) == 2                                # the prompt step and the decode step
    for layout in plans:
        arena = layout.arena
        assert arena.bytes_saved() > 0 and arena.regions() < len(arena)
        assert arena.arena_bytes < arena.bytes_without_sharing()
    assert session.workspace.bytes() == max(256, max(l.arena.arena_bytes for l in plans))
    report = session.workspace_report()
    assert report["held_bytes"] == session.workspace.bytes() and len(report["plans"]) == 2
    assert all(p["bytes_saved"] == p["bytes_without_sharing"] - p["arena_bytes"] > 0
               for p in report["plans"].values())
    # a step that wants no logits plans none (runtime/tests/decoder_output_plan_test.cpp:11-41)
    slot = session.begin()
    for _ in range(2):
        assert session.step([(slot, prompts[0][:7], [])]).shape == (0, 381)
    silent = [l.arena for sig, l in session.workspace._plans.items() if sig[2] == 0]
    assert len(silent) == 1 and not any(name.startswith("logits") for name in silent[0].names())
    assert any(name.startswith("logits") for name in plans[0].arena.names())


def test_a_failed_step_leaves_the_session_as_it_was_and_a_failed_wait_ends_it(models, references,
                                                                              monkeypatch):
    """The failure contract (runtime/src/qwen3.cpp:126-161,374-379 of the reference), with the
    failures forced from the host: an error inside a step is raised as it is, the sequences
    keep their lengths and go on correctly afterwards; if even waiting for the launched work
    fails, the session refuses every later call."""
    import edge_infer_amd as ei
    model = models("A", "float32")
    session = ei.Session(model, max_tokens=512, max_seqs=2)
    ids = requests_for("A", LENGTHS["A"])[0]
    ref = references["A"][0]
    slot = session.begin()
    session.step([(slot, ids[:40], [])])
    real_forward = model.forward
    calls = []

    def failing(ctx):
        calls.append(ctx.n_rows)
        real_forward(ctx)                          # the work is launched, then the step fails
        raise FloatingPointError("forced")
    monkeypatch.setattr(model, "forward", failing)
    for tokens in (ids[40:50], ids[40:41]):        # a prompt chunk and a decode step
        with pytest.raises(FloatingPointError, match="forced"):
            session.step([(slot, tokens, [0])])
        assert session.length(slot) == 40
    monkeypatch.setattr(model, "forward", real_forward)
    logits = session.step([(slot, ids[40:50], list(range(10)))])
    assert_close("float32", logits, ref[40:50], "after failed steps")
    out = session.step([(slot, ids[50:51], [0])])
    assert_close("float32", out, ref[50:51], "decode after failed steps")
    # the wait fails as well: unusable for good
    monkeypatch.setattr(model, "forward", failing)

    def no_sync(device=None):
        raise RuntimeError("forced sync failure")
    monkeypatch.setattr(torch.cuda, "synchronize", no_sync)
    with pytest.raises(FloatingPointError, match="forced"):
        session.step([(slot, ids[51:53], [0])])     # (two tokens: a single one would replay a graph)
    monkeypatch.undo()
    for call in (lambda: session.step([(slot, ids[51:52], [0])]), session.begin, session.reset,
                 lambda: session.generate([1, 2, 3])):
        with pytest.raises(RuntimeError, match="unusable"):
            call()
    torch.cuda.synchronize()


# What the bfloat16 engine may differ by from the float32 engine on 8 and on all 36 layers of
# the 8B shape with the real vocabulary: root-mean-square difference / root-mean-square logit,
# largest difference / largest logit, the share of logits within the reference's bound (below)
# and the share of places with the same most likely token.  Measured on an MI355X at 8 layers:
# 0.0173, 0.0197, 73.7 %, 92.2 % (about 0.2 % of rounding error per operation, ten roundings a
# layer, adding up like a random walk: the square root of the depth); at 36 layers: 0.0358,
# 0.0417, 42.9 %, 96.9 %.  Random weights give logits of at most 0.6, so the absolute part of
# the reference's bound, made for trained weights, decides less the deeper the model is.
DEPTH_BOUNDS = {8: (0.02, 0.03, 0.70, 0.85),
                36: (0.042, 0.05, 0.38, 0.85)}


@pytest.mark.parametrize("layers", [8, 36])
def test_bfloat16_against_float32_at_depth_on_the_8b_shape(layers):
    """The two precisions of the whole engine at real width and vocabulary, deeper than
    the tiny models: 300- and 120-token prompts, then 24 tokens one by one each.  Reported
    and bounded: rms and largest difference, the share of logits within the reference's
    bound |a - r| <= 0.015625 + 0.01 max(|a|, |r|) (runtime/tests/qwen3_session_test.cpp:325-326,
    there for its two-layer test model), and how often the top token is the same.  Random
    weights make nearly flat logits (the top two are often closer than bfloat16 resolves),
    so equal top tokens everywhere cannot be asked for; where they differ the float32
    engine's own margin between the two must be small."""
    import edge_infer_amd as ei
    cfg = ei.Qwen3Config(vocab_size=151936, hidden_size=4096, num_hidden_layers=layers,
                         num_attention_heads=32, num_key_value_heads=8, head_dim=128,
                         intermediate_size=12288, max_position_embeddings=1024, bos_token_id=0,
                         eos_token_id=151645, rms_norm_eps=1e-6, rope_theta=1e6,
                         tie_word_embeddings=False)
    prompts = [random_ids(cfg.vocab_size, 300, 41), random_ids(cfg.vocab_size, 120, 42)]
    feed = [random_ids(cfg.vocab_size, 24, 43), random_ids(cfg.vocab_size, 24, 44)]

    def run(dtype):
        model = ei.random_model(cfg, seed=2, dtype=dtype)
        session = ei.Session(model, max_tokens=1024, max_seqs=2)
        slots = [session.begin(), session.begin()]
        rows = [session.step([(s, p, list(range(len(p) - 8, len(p))))
                              for s, p in zip(slots, prompts)])]
        for t in range(24):
            rows.append(session.step([(s, [f[t]], [0]) for s, f in zip(slots, feed)]))
        assert session.graph_replays > 0
        out = torch.cat(rows).double().cpu()
        del session, model
        torch.cuda.empty_cache()
        return out

    exact, low = run("float32"), run("bfloat16")
    assert exact.shape == (16 + 48, cfg.vocab_size)
    diff = (low - exact).abs()
    rms = diff.pow(2).mean().sqrt().item() / exact.pow(2).mean().sqrt().item()
    worst = diff.max().item() / exact.abs().max().item()
    within = (diff <= 0.015625 + 0.01 * torch.maximum(low.abs(), exact.abs())).double().mean().item()
    same = (low.argmax(-1) == exact.argmax(-1)).double().mean().item()
    print(f"\nbfloat16 against float32, {layers} layers of the 8B shape: rms {rms:.4f}, "
          f"max {worst:.4f}, within the reference's bound {within:.4f}, same top token {same:.3f}")
    rms_bound, max_bound, within_bound, same_bound = DEPTH_BOUNDS[layers]
    assert rms <= rms_bound and worst <= max_bound
    assert within >= within_bound and same >= same_bound
    # where the top token differs, float32 itself holds the two within bfloat16's error
    for row in (low.argmax(-1) != exact.argmax(-1)).nonzero().flatten().tolist():
        margin = exact[row].max() - exact[row, low[row].argmax()]
        assert margin <= 2 * diff[row].max(), f"place {row}: margin {margin:.4f}"


def head64_folder(root):
    """A model whose bfloat16 steps take the matrix-core attention kernels (head size 64),
    the decode kernel that writes the position's key and value itself included."""
    import edge_infer_amd as ei
    cfg = ei.Qwen3Config(vocab_size=500, hidden_size=128, num_hidden_layers=2,
                         num_attention_heads=4, num_key_value_heads=2, head_dim=64,
                         intermediate_size=256, max_position_embeddings=512, bos_token_id=1,
                         eos_token_id=499, rms_norm_eps=1e-6, rope_theta=1e4,
                         tie_word_embeddings=True)
    return ei.write_model_folder(root / "head64", cfg, seed=5)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("which", ["B", "head64"])
def test_a_step_writes_only_its_own_positions_of_the_cache(folders, tmp_path, which, dtype):
    """The whole cache is filled with a sentinel; after every step exactly the positions
    [old length, new length) of the stepped slots have changed, in every layer's keys and
    values, and nothing else: not the rest of their pages, not other slots, not free pages,
    not what a padding row of a captured step points at
    (runtime/tests/qwen3_session_test.cpp:174-185,309-319 holds the same for its one slot)."""
    import edge_infer_amd as ei
    folder = folders["B"] if which == "B" else head64_folder(tmp_path)
    model = ei.load_model(folder, dtype=dtype)
    vocab = model.spec.vocab_size
    session = ei.Session(model, max_tokens=12 * 64, max_seqs=4)
    assert session.graphs
    cache = session.cache
    sentinel = -123.0
    for tensor in cache.kv_k + cache.kv_v:
        tensor.fill_(sentinel)

    def stepped(entries):
        before = [t.clone() for t in cache.kv_k + cache.kv_v]
        old = {slot: session.length(slot) for slot, _, _ in entries}
        session.step(entries)
        torch.cuda.synchronize()
        for group, pages in enumerate(cache.kv_pages):
            expected = torch.zeros(cache.kv_k[group].shape[1:4:2], dtype=torch.bool)  # [page, 64]
            for slot, tokens, _ in entries:
                row = pages.row(slot)
                for pos in range(old[slot], old[slot] + len(tokens)):
                    expected[row[pos // 64], pos % 64] = True
            for name, now, was in (("k", cache.kv_k[group], before[group]),
                                   ("v", cache.kv_v[group], before[len(cache.kv_k) + group])):
                changed = (now != was).cpu()             # [entry, page, kv head, 64, d]
                assert torch.equal(changed.any(dim=-1).any(dim=2).any(dim=0), expected), \
                    f"{name}: positions written differ from the step's own"
                # ... and there every layer, head and element was written
                written = (now != sentinel).cpu().all(dim=-1).all(dim=2).all(dim=0)
                assert bool(written[expected].all()), name

    a, b, c = (random_ids(vocab, n, 60 + i) for i, n in enumerate((130, 9, 70)))
    sa, sb, sc = session.begin(), session.begin(), session.begin()
    stepped([(sa, a[:100], [99]), (sb, b[:5], []), (sc, c[:64], [0, 63])])   # unequal prompts
    stepped([(sa, a[100:101], [0]), (sb, b[5:6], [0]), (sc, c[64:65], [0])])  # eager, then captured
    stepped([(sa, a[101:102], [0]), (sb, b[6:7], [0]), (sc, c[65:66], [0])])  # replayed, one padding row
    assert session.graph_replays == 1
    stepped([(sa, a[102:129], [26])])                                         # a portion of 27
    session.end(sb)
    sd = session.begin()                 # the slot again, with other tokens than it held
    stepped([(sd, random_ids(vocab, 9, 99), [8]), (sc, c[66:70], [3])])
    stepped([(sa, a[129:130], [0])])
    session.cache.check()


@pytest.mark.parametrize("dtype", DTYPES)
def test_steady_decoding_allocates_nothing_on_the_device(folders, tmp_path, dtype):
    """After the first steps of a batch have captured their graph, fifty more decode steps
    (greedy sampling and the copy of the tokens included) ask the device allocator for
    nothing (runtime/tests/qwen3_session_test.cpp:469-531 counts allocations the same way)."""
    import edge_infer_amd as ei
    from edge_infer_amd.sampling import Sampler, SamplingParams
    model = ei.load_model(head64_folder(tmp_path), dtype=dtype)
    session = ei.Session(model, max_tokens=4 * 256, max_seqs=4, max_seq_tokens=256)
    sampler, greedy = Sampler(model.device), SamplingParams(temperature=0.0)
    prompts = [random_ids(500, n, 80 + n) for n in (40, 3, 17)]
    slots = [session.begin() for _ in prompts]
    logits = session.step([(s, p, [len(p) - 1]) for s, p in zip(slots, prompts)], copy=False)
    tokens = sampler(logits, greedy, [], [])

    def decode(count):
        nonlocal tokens
        for _ in range(count):
            logits = session.step([(s, [t], [0]) for s, t in zip(slots, tokens)], copy=False)
            tokens = sampler(logits, greedy, [], [])
    decode(3)
    torch.cuda.synchronize()
    stats = torch.cuda.memory_stats()
    before = (stats["allocation.all.allocated"], stats["segment.all.allocated"],
              stats["allocated_bytes.all.current"], stats["reserved_bytes.all.current"])
    replays = session.graph_replays
    decode(50)
    torch.cuda.synchronize()
    stats = torch.cuda.memory_stats()
    after = (stats["allocation.all.allocated"], stats["segment.all.allocated"],
             stats["allocated_bytes.all.current"], stats["reserved_bytes.all.current"])
    assert after == before, f"allocator figures moved: {before} -> {after}"
    assert session.graph_replays == replays + 50


@pytest.mark.parametrize("dtype", DTYPES)
def test_prompts_in_portions_give_the_logits_of_whole_prompts(tmp_path, dtype):
    """The generation loop's prompt steps under a row budget of 64: a prompt cut at 64 and
    128, a portion of 2 tokens that begins a page (positions 64 and 65), requests that are
    left out of a step, at head size 64 (the matrix-core kernels in bfloat16), against whole
    prompts in the plain implementation."""
    import edge_infer_amd as ei
    from edge_infer_amd.engine.generate import Request, _prefill, prompt_steps
    folder = head64_folder(tmp_path)
    cfg, w = plain.read_folder(folder)
    prompts = [random_ids(500, n, 30 + n) for n in (66, 5, 130, 33, 52)]
    session = ei.Session(ei.load_model(folder, dtype=dtype), max_tokens=8 * 192, max_seqs=5)
    requests = [Request(prompt=p, limit=200, stream=i) for i, p in enumerate(prompts)]
    portions = [[(r.stream, first, count) for r, first, count, _ in step]
                for step in prompt_steps(requests, 64)]
    assert portions == [[(0, 0, 64)], [(0, 64, 2), (1, 0, 5), (2, 0, 57)], [(2, 57, 64)],
                        [(2, 121, 9), (3, 0, 33), (4, 0, 22)], [(4, 22, 30)]]
    for request in requests:
        request.slot = session.begin()
    logits = _prefill(session, requests, 64)
    expected = torch.stack([plain.forward(w, cfg, p)[-1] for p in prompts])
    assert_close(dtype, logits, expected, f"{dtype} prompts in portions")
    assert [session.length(r.slot) for r in requests] == [66, 5, 130, 33, 52]
    # and through the whole loop: the same tokens as with one prompt step
    session.reset()
    few = session.generate_batch(prompts, max_new_tokens=5, temperature=0.0, stop_ids=(),
                                 prompt_rows=64)
    if dtype == "float32":
        assert few == [plain.generate(w, cfg, p, max_length=len(p) + 5, stop_ids=set())
                       for p in prompts]
    assert [len(tokens) for tokens in few] == [5] * 5
