"""The plain implementation is pinned by what fixes it beside the reference's text:
vectors that the reference's own tests hold, special cases that reduce to a library
routine, and invariants.  Each check fails for a plausible mistake (named in its
docstring)."""
import math

import numpy as np
import pytest
import torch
import torch.nn.functional as F

import plain_qwen3 as plain
from helpers import CONFIGS

torch.manual_seed(0)


def test_rms_norm_reference_vector():
    """operators/tests/operators_cuda_bf16_contract_test.cu:235-284: x_i = -0.8 + 0.25 (i mod 7),
    w_i = 0.63 + 0.17 (i mod 5), width 128, eps 1e-6; expected (x * inv) * w with
    inv = 1 / sqrt(sum / n + eps).  Fails for a `1 + w` weight or a missing eps."""
    n = 128
    x = np.array([-0.8 + (i % 7) * 0.25 for i in range(n)], dtype=np.float32)
    w = np.array([0.63 + (i % 5) * 0.17 for i in range(n)], dtype=np.float32)
    inv = 1.0 / math.sqrt(float((x.astype(np.float64) ** 2).sum()) / n + 1e-6)
    expected = x.astype(np.float64) * inv * w.astype(np.float64)
    got = plain.rms_norm(torch.from_numpy(x), torch.from_numpy(w), 1e-6).numpy()
    assert np.abs(got - expected).max() < 2e-6   # the reference's own bound
    assert np.abs(got - x * inv * (1 + w)).max() > 0.1


def test_rms_norm_library_and_invariants():
    x = torch.randn(5, 48, dtype=torch.float64)
    w = torch.randn(48, dtype=torch.float64)
    expected = x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + 1e-5) * w
    assert torch.allclose(plain.rms_norm(x, w, 1e-5), expected, atol=1e-12)
    # scaling the row changes nothing when eps vanishes; constant rows become +-1
    assert torch.allclose(plain.rms_norm(3.7 * x, w, 1e-30), plain.rms_norm(x, w, 1e-30), atol=1e-9)
    ones = plain.rms_norm(torch.full((1, 8), -2.5), torch.ones(8), 1e-30)
    assert torch.allclose(ones, -torch.ones(1, 8, dtype=torch.float64), atol=1e-9)
    # eps sits inside the root, next to the mean (not added to the root)
    tiny = plain.rms_norm(torch.full((1, 4), 1e-4, dtype=torch.float64), torch.ones(4), 1e-2)
    assert abs(tiny[0, 0].item() - 1e-4 / math.sqrt(1e-8 + 1e-2)) < 1e-12


def test_linear_is_x_times_w_transposed():
    """Rectangular so that a missing transpose cannot pass."""
    x = torch.randn(3, 7, dtype=torch.float64)
    w = torch.randn(11, 7, dtype=torch.float64)
    assert torch.allclose(plain.linear(x, w), F.linear(x, w), atol=1e-12)
    assert plain.linear(x, w).shape == (3, 11)


def test_rope_small_angle_reference_vector():
    """operators/tests/operators_cuda_bf16_contract_test.cu:372-415: basis (1,..,1,0,..,0),
    theta 1e6, positions 0..20 give (cos, sin) of the float64 angle in the two halves.
    Fails for interleaved pairs, a wrong sign of the sine, or theta^(+2i/d)."""
    d = 128
    basis = torch.zeros(21, 1, d, dtype=torch.float64)
    basis[..., :d // 2] = 1.0
    out = plain.rope(basis, list(range(21)), 1e6)
    for p in range(21):
        for i in range(d // 2):
            angle = p / (1e6 ** (2.0 * i / d))
            assert abs(out[p, 0, i].item() - math.cos(angle)) < 2e-6
            assert abs(out[p, 0, i + d // 2].item() - math.sin(angle)) < 2e-6


def test_rope_position_three_reference_vector():
    """operators/tests/operators_cuda_bf16_contract_test.cu:328-370 without its bfloat16
    staging: position 3, theta 1e4, x_i = -1.23 + 0.173 (i mod 19), width 128."""
    d = 128
    x = np.array([-1.23 + (i % 19) * 0.173 for i in range(d)], dtype=np.float64)
    out = plain.rope(torch.from_numpy(x).reshape(1, 1, d), [3], 1e4)[0, 0].numpy()
    for i in range(d // 2):
        angle = 3.0 / (1e4 ** (2.0 * i / d))
        c, s = math.cos(angle), math.sin(angle)
        assert abs(out[i] - (x[i] * c - x[i + d // 2] * s)) < 1e-5
        assert abs(out[i + d // 2] - (x[i] * s + x[i + d // 2] * c)) < 1e-5


def test_rope_invariants():
    d = 32
    q = torch.randn(1, 1, d, dtype=torch.float64)
    k = torch.randn(1, 1, d, dtype=torch.float64)
    # position 0 is the identity
    assert torch.allclose(plain.rope(q, [0], 1e4), q, atol=1e-12)
    # each pair (i, i + d/2) keeps its norm
    r = plain.rope(q, [37], 1e4)
    assert torch.allclose(r[..., :d // 2] ** 2 + r[..., d // 2:] ** 2,
                          q[..., :d // 2] ** 2 + q[..., d // 2:] ** 2, atol=1e-12)
    # q(p) . k(p') depends on p - p' only (angles are float32, hence the tolerance)
    a = (plain.rope(q, [9], 1e4) * plain.rope(k, [4], 1e4)).sum()
    b = (plain.rope(q, [25], 1e4) * plain.rope(k, [20], 1e4)).sum()
    assert abs(a - b) < 1e-5
    c = (plain.rope(q, [9], 1e4) * plain.rope(k, [5], 1e4)).sum()
    assert abs(a - c) > 1e-3
    # equals the complex product (x + iy) e^{i p f}
    z = torch.complex(q[0, 0, :d // 2], q[0, 0, d // 2:])
    f = torch.tensor([1.0 / (1e4 ** (2.0 * i / d)) for i in range(d // 2)], dtype=torch.float64)
    rotated = z * torch.exp(1j * 37 * f)
    assert torch.allclose(r[0, 0, :d // 2], rotated.real, atol=1e-5)
    assert torch.allclose(r[0, 0, d // 2:], rotated.imag, atol=1e-5)


def test_attention_equals_library_routine():
    """Plain causal attention without groups is F.scaled_dot_product_attention."""
    S, h, d = 9, 3, 16
    q, k, v = (torch.randn(S, h, d, dtype=torch.float64) for _ in range(3))
    expected = F.scaled_dot_product_attention(q.transpose(0, 1), k.transpose(0, 1),
                                              v.transpose(0, 1), is_causal=True).transpose(0, 1)
    assert torch.allclose(plain.attention(q, k, v), expected, atol=1e-10)


def test_attention_special_cases():
    S, nq, nkv, d = 7, 4, 2, 16
    q = torch.randn(S, nq, d, dtype=torch.float64)
    k = torch.randn(S, nkv, d, dtype=torch.float64)
    v = torch.randn(S, nkv, d, dtype=torch.float64)
    out = plain.attention(q, k, v)
    # the first position sees one key: its output is that value (consecutive heads share)
    for h in range(nq):
        assert torch.allclose(out[0, h], v[0, h // (nq // nkv)], atol=1e-12)
    # identical keys: the mean of the visible values
    same = plain.attention(q, k[:1].expand(S, -1, -1), v)
    assert torch.allclose(same[4, 1], v[:5, 0].mean(0), atol=1e-12)
    # grouped heads equal full heads with every kv head repeated nq/nkv times
    full = plain.attention(q, k.repeat_interleave(nq // nkv, 1), v.repeat_interleave(nq // nkv, 1))
    assert torch.allclose(out, full, atol=1e-12)
    # a window of 3 sees the last three keys only
    w = plain.attention(q, k, v, window=3)
    manual = plain.attention(q[3:6], k[3:6], v[3:6])
    assert torch.allclose(w[5], manual[2], atol=1e-12)
    assert not torch.allclose(w[5], out[5], atol=1e-6)


def test_swiglu_and_silu():
    g = torch.tensor([-88.0, -3.0, 0.0, 0.5, 20.0], dtype=torch.float64)
    u = torch.tensor([2.0, -1.0, 4.0, 3.0, 0.5], dtype=torch.float64)
    assert torch.allclose(plain.swiglu(g, u), F.silu(g) * u, atol=1e-12)
    assert plain.silu(torch.tensor([0.0]))[0] == 0
    assert abs(plain.silu(torch.tensor([30.0]))[0] - 30.0) < 1e-9
    assert torch.isfinite(plain.silu(torch.tensor([-88.0]))).all()   # the reference's tail case


def _random_weights(cfg, seed):
    g = torch.Generator().manual_seed(seed)
    H, V, I = cfg["hidden_size"], cfg["vocab_size"], cfg["intermediate_size"]
    d = plain.head_dim_of(cfg)
    Q, KV = cfg["num_attention_heads"] * d, cfg["num_key_value_heads"] * d
    def mat(*shape):
        return (torch.randn(*shape, generator=g) * 0.05).double()
    def nrm(n):
        return (1 + (torch.rand(n, generator=g) * 0.2 - 0.1)).double()
    w = {"model.embed_tokens.weight": mat(V, H), "model.norm.weight": nrm(H)}
    if not cfg.get("tie_word_embeddings", False):
        w["lm_head.weight"] = mat(V, H)
    for i in range(cfg["num_hidden_layers"]):
        p = f"model.layers.{i}."
        w[p + "input_layernorm.weight"] = nrm(H)
        w[p + "post_attention_layernorm.weight"] = nrm(H)
        w[p + "self_attn.q_proj.weight"] = mat(Q, H)
        w[p + "self_attn.k_proj.weight"] = mat(KV, H)
        w[p + "self_attn.v_proj.weight"] = mat(KV, H)
        w[p + "self_attn.o_proj.weight"] = mat(H, Q)
        w[p + "self_attn.q_norm.weight"] = nrm(d)
        w[p + "self_attn.k_norm.weight"] = nrm(d)
        w[p + "mlp.gate_proj.weight"] = mat(I, H)
        w[p + "mlp.up_proj.weight"] = mat(I, H)
        w[p + "mlp.down_proj.weight"] = mat(H, I)
    return w


def test_one_layer_one_head_model_is_a_straight_line_of_library_calls():
    """One layer, one head, no grouping: the whole model written once more with
    torch's own routines.  Fails when a norm sits in the wrong place (after the
    rotation, or the post-attention norm before the residual sum)."""
    cfg = dict(vocab_size=50, hidden_size=24, num_hidden_layers=1, num_attention_heads=1,
               num_key_value_heads=1, head_dim=16, intermediate_size=40, rms_norm_eps=1e-6,
               rope_theta=1e4, tie_word_embeddings=False, eos_token_id=49)
    w = _random_weights(cfg, 3)
    ids = [3, 17, 9, 44, 0, 21]
    p = "model.layers.0."
    def norm(x, weight):
        return x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + 1e-6) * weight
    x = F.embedding(torch.tensor(ids), w["model.embed_tokens.weight"])
    h = norm(x, w[p + "input_layernorm.weight"])
    q = norm(F.linear(h, w[p + "self_attn.q_proj.weight"]), w[p + "self_attn.q_norm.weight"])
    k = norm(F.linear(h, w[p + "self_attn.k_proj.weight"]), w[p + "self_attn.k_norm.weight"])
    v = F.linear(h, w[p + "self_attn.v_proj.weight"])
    q = plain.rope(q[:, None, :], range(len(ids)), 1e4)[:, 0]
    k = plain.rope(k[:, None, :], range(len(ids)), 1e4)[:, 0]
    a = F.scaled_dot_product_attention(q[None], k[None], v[None], is_causal=True)[0]
    x = x + F.linear(a, w[p + "self_attn.o_proj.weight"])
    h = norm(x, w[p + "post_attention_layernorm.weight"])
    x = x + F.linear(F.silu(F.linear(h, w[p + "mlp.gate_proj.weight"]))
                     * F.linear(h, w[p + "mlp.up_proj.weight"]), w[p + "mlp.down_proj.weight"])
    expected = F.linear(norm(x, w["model.norm.weight"]), w["lm_head.weight"])
    assert torch.allclose(plain.forward(w, cfg, ids), expected, atol=1e-10)


@pytest.mark.parametrize("name", ["A", "B"])
def test_model_invariants(name):
    cfg = dict(CONFIGS[name])
    w = _random_weights(cfg, 7)
    ids = [5, 3, 8, 13, 2, 1, 34, 21]
    logits = plain.forward(w, cfg, ids)
    # causal: a prefix gives the same rows
    assert torch.allclose(plain.forward(w, cfg, ids[:5]), logits[:5], atol=1e-10)
    # only distances count: shifting every position changes nothing (beyond float32 angles)
    shifted = plain.forward(w, cfg, ids, positions=[p + 40 for p in range(len(ids))])
    assert (shifted - logits).abs().max() < 1e-4 * logits.abs().max()
    moved = plain.forward(w, cfg, ids, positions=[2 * p for p in range(len(ids))])
    assert (moved - logits).abs().max() > 1e-3 * logits.abs().max()
    # a tied head is the embedding used as the head
    tied = dict(cfg, tie_word_embeddings=True)
    wt = {k: v for k, v in w.items() if k != "lm_head.weight"}
    wu = dict(wt, **{"lm_head.weight": wt["model.embed_tokens.weight"].clone()})
    assert torch.equal(plain.forward(wt, tied, ids), plain.forward(wu, dict(cfg, tie_word_embeddings=False), ids))


def test_sampling_reference_distribution():
    """operators/tests/operators_cuda_sampling_test.cu:70-101,144-198: logits log{.4,.3,.2,.1},
    (T, p, k) in {(1,1,2), (1,.65,4), (.75,.95,3)}: support, probabilities, frequencies."""
    logits = np.log(np.array([0.4, 0.3, 0.2, 0.1], dtype=np.float32))
    def reference(temperature, top_p, top_k):
        order = [0, 1, 2, 3]
        prob = [0.0] * 4
        k = min(top_k, 4)
        total = 0.0
        for i in range(k):
            prob[order[i]] = math.exp((float(logits[order[i]]) - float(logits[order[0]])) / temperature)
            total += prob[order[i]]
        kept, cumulative = 0, 0.0
        while True:
            cumulative += prob[order[kept]]
            kept += 1
            if not (kept < k and cumulative < top_p * total):
                break
        for i in range(kept, 4):
            prob[order[i]] = 0.0
        return [p / cumulative for p in prob]
    for temperature, top_p, top_k in [(1.0, 1.0, 2), (1.0, 0.65, 4), (0.75, 0.95, 3)]:
        expected = reference(temperature, top_p, top_k)
        order, prob = plain.filtered_distribution(logits, temperature, top_p, top_k)
        for token, p in zip(order, prob):
            assert abs(p - expected[token]) < 2e-5
        assert all(expected[t] > 0 for t in order) and len(order) == sum(p > 0 for p in expected)
        counts = [0] * 4
        for draw in range(2048):
            counts[plain.sample(logits, temperature, top_p, top_k, plain.uniform(1234567, 0, draw))] += 1
        assert max(abs(c / 2048 - e) for c, e in zip(counts, expected)) < 0.05


def test_sampling_greedy_and_ties():
    """operators_cuda_sampling_test.cu:103-131: rows (2,1,0,-1), (-3,5,1,0), (0,-1,4,2) -> 0, 1, 2
    for (T=1, k=1) and (T=0, k=4); equal logits go to the lowest index."""
    rows = [[2, 1, 0, -1], [-3, 5, 1, 0], [0, -1, 4, 2]]
    for temperature, top_k in [(1.0, 1), (0.0, 4)]:
        assert [plain.sample(r, temperature, 1.0, top_k, 0.5) for r in rows] == [0, 1, 2]
    assert plain.sample([1.0, 3.0, 3.0, 2.0], 0.0, 1.0, 1, 0.5) == 1
    assert plain.sample([float("nan"), 1.0], 0.0, 1.0, 1, 0.5) == 1
    # u = 1 selects the last kept element, a tiny u the first
    assert plain.sample([0.0, 0.0, 0.0], 1.0, 1.0, 3, 1.0) == 2
    assert plain.sample([0.0, 0.0, 0.0], 1.0, 1.0, 3, 1e-7) == 0


def test_uniform_is_in_range_and_keyed():
    draws = [plain.uniform(7, s, c) for s in range(4) for c in range(64)]
    assert all(0.0 < u <= 1.0 for u in draws)
    assert len(set(draws)) > 250
    assert plain.uniform(7, 1, 2) == plain.uniform(7, 1, 2) != plain.uniform(8, 1, 2)
    assert abs(sum(draws) / len(draws) - 0.5) < 0.06


def test_generate_rules():
    """runtime/src/inference.cpp:367-418: max_length counts the prompt; a limit that does not
    exceed the prompt yields nothing; the stop token is not returned."""
    cfg = dict(CONFIGS["A"])
    w = _random_weights(cfg, 11)
    prompt = [1, 2, 3, 4]
    assert plain.generate(w, cfg, prompt, max_length=4) == []
    out = plain.generate(w, cfg, prompt, max_length=9, stop_ids=set())
    assert len(out) == 5
    again = plain.generate(w, cfg, prompt, max_length=9, stop_ids={out[2]})
    assert again == out[:out.index(out[2])]


def test_linear_bias_is_added_to_every_row():
    """operators/src/cuda/execution.cu:61-66,307-317: the bias row initialises the product."""
    g = torch.Generator().manual_seed(3)
    x, w, b = (torch.randn(shape, generator=g, dtype=torch.float64)
               for shape in ((5, 7), (3, 7), (3,)))
    expected = torch.nn.functional.linear(x, w, b)
    assert torch.allclose(plain.linear(x, w, b), expected, atol=1e-12)
    assert torch.allclose(plain.linear(x, w, b) - plain.linear(x, w), b.expand(5, 3), atol=1e-12)


# ----------------------------------------------------------------------------
# the composition: what fixes the order of the parts beside the reference's text
# ----------------------------------------------------------------------------
def _wide_head_norms(w, cfg, seed):
    """q/k norm weights far from 1 and different in the two halves of every rotation pair:
    only then does their place relative to the rotation show."""
    g = torch.Generator().manual_seed(seed)
    d = plain.head_dim_of(cfg)
    for i in range(cfg["num_hidden_layers"]):
        for name in ("q_norm", "k_norm"):
            w[f"model.layers.{i}.self_attn.{name}.weight"] = \
                (0.4 + 2.0 * torch.rand(d, generator=g)).double()
    return w


def _attention_block_with_the_norm_after_the_rotation(x, w, cfg, layer, positions):
    """The mistake that the shift test below must catch: rotation first, head norm second."""
    p = f"model.layers.{layer}."
    S = x.shape[0]
    nq, nkv, d = cfg["num_attention_heads"], cfg["num_key_value_heads"], plain.head_dim_of(cfg)
    h = plain.rms_norm(x, w[p + "input_layernorm.weight"], cfg["rms_norm_eps"])
    q = plain.linear(h, w[p + "self_attn.q_proj.weight"]).reshape(S, nq, d)
    k = plain.linear(h, w[p + "self_attn.k_proj.weight"]).reshape(S, nkv, d)
    v = plain.linear(h, w[p + "self_attn.v_proj.weight"]).reshape(S, nkv, d)
    q = plain.rms_norm(plain.rope(q, positions, cfg["rope_theta"]),
                       w[p + "self_attn.q_norm.weight"], cfg["rms_norm_eps"])
    k = plain.rms_norm(plain.rope(k, positions, cfg["rope_theta"]),
                       w[p + "self_attn.k_norm.weight"], cfg["rms_norm_eps"])
    a = plain.attention(q, k, v, positions)
    return plain.linear(a.reshape(S, nq * d), w[p + "self_attn.o_proj.weight"])


@pytest.mark.parametrize("name", ["A", "B"])
def test_only_distances_count_because_the_head_norm_precedes_the_rotation(name, monkeypatch):
    """A rotation commutes with nothing that weighs the two halves of a pair differently, so
    with head norm weights far from 1 the logits are free of a common shift of all positions
    only if the norm comes before the rotation (runtime/include/execution/decoder.hpp:125-136).
    The same model with the two exchanged moves by a hundred times the bound."""
    cfg = dict(CONFIGS[name])
    w = _wide_head_norms(_random_weights(cfg, 21), cfg, 22)
    # larger projections, so that attention is far from uniform and the keys matter
    for key in list(w):
        if "q_proj" in key or "k_proj" in key:
            w[key] = w[key] * 8
    ids = [5, 3, 8, 13, 2, 1, 34, 21, 7, 7, 19]
    shift = [p + 57 for p in range(len(ids))]
    logits = plain.forward(w, cfg, ids)
    scale = logits.abs().max()
    assert (plain.forward(w, cfg, ids, positions=shift) - logits).abs().max() < 1e-4 * scale
    monkeypatch.setattr(plain, "attention_block", _attention_block_with_the_norm_after_the_rotation)
    wrong = plain.forward(w, cfg, ids)
    assert (plain.forward(w, cfg, ids, positions=shift) - wrong).abs().max() > 1e-2 * wrong.abs().max()


def test_with_silent_blocks_the_model_is_embedding_final_norm_and_head():
    """o_proj = down_proj = 0 in every layer: what is left is head(norm(E[ids]) * w), from
    library routines.  Fails for a scaled embedding, a final norm without its weight or
    applied to the head's output, a residual that is not carried through, or a bias that
    does not exist."""
    cfg = dict(CONFIGS["B"])
    w = _random_weights(cfg, 5)
    for key in list(w):
        if "o_proj" in key or "down_proj" in key:
            w[key] = torch.zeros_like(w[key])
    ids = [7, 300, 12, 12, 0]
    x = F.embedding(torch.tensor(ids), w["model.embed_tokens.weight"])
    y = x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + cfg["rms_norm_eps"]) * w["model.norm.weight"]
    assert torch.allclose(plain.forward(w, cfg, ids), F.linear(y, w["lm_head.weight"]), atol=1e-12)


def _dominant_attention_model(seed):
    """One layer, one head, made so that the feed-forward's input shows where its norm sits.

    Every row of v_proj is the same vector, so attention's output is a scalar times (1,..,1);
    o_proj sends that to s * scalar * e_0 with s = 1e9, which buries the embedding: the
    residual after attention points along +-e_0 at every position, whatever the token.  The
    second norm of a sequential block therefore hands the feed-forward +-sqrt(H) w2[0] e_0,
    the same input (up to the sign) at every position.  down_proj writes with the same scale
    s and never into coordinate 0; the head is the identity and the final norm's weight 1, so
    the logits are the normalised residual and their part beyond coordinate 0 points along
    the feed-forward's output."""
    cfg = dict(vocab_size=24, hidden_size=24, num_hidden_layers=1, num_attention_heads=1,
               num_key_value_heads=1, head_dim=16, intermediate_size=40, rms_norm_eps=1e-30,
               rope_theta=1e4, tie_word_embeddings=False, eos_token_id=23)
    w = _random_weights(cfg, seed)
    H, d, s = cfg["hidden_size"], 16, 1e9
    p = "model.layers.0."
    w[p + "self_attn.v_proj.weight"] = w[p + "self_attn.v_proj.weight"][:1].expand(d, H).clone()
    o = torch.zeros(H, d, dtype=torch.float64)
    o[0, :] = s / d
    w[p + "self_attn.o_proj.weight"] = o
    down = w[p + "mlp.down_proj.weight"] * s * 10
    down[0, :] = 0
    w[p + "mlp.down_proj.weight"] = down
    w[p + "mlp.gate_proj.weight"] = w[p + "mlp.gate_proj.weight"] * 10
    w["model.norm.weight"] = torch.ones(H, dtype=torch.float64)
    w["lm_head.weight"] = torch.eye(H, dtype=torch.float64)
    return cfg, w


def test_the_second_norm_reads_the_residual_after_attention_was_added():
    """runtime/include/execution/decoder.hpp:159-161: the feed-forward's norm reads the sum.
    In the model above its output is then one of two vectors, from library routines:
    down(silu(c gate[:, 0]) * c up[:, 0]) with c = +-sqrt(H) w2[0].  A block whose second
    norm read the residual before attention's addition (or the embedding) would give a
    different direction at every position."""
    cfg, w = _dominant_attention_model(13)
    p = "model.layers.0."
    ids = [3, 17, 9, 21, 0, 11, 5, 5, 14]
    logits = plain.forward(w, cfg, ids)
    H = cfg["hidden_size"]
    c = math.sqrt(H) * w[p + "post_attention_layernorm.weight"][0]
    candidates = []
    for sign in (1.0, -1.0):
        hidden = F.silu(sign * c * w[p + "mlp.gate_proj.weight"][:, 0]) \
            * (sign * c * w[p + "mlp.up_proj.weight"][:, 0])
        delta = F.linear(hidden, w[p + "mlp.down_proj.weight"])[1:]
        candidates.append(delta / delta.norm())
    assert (candidates[0] - candidates[1]).norm() > 0.1     # the two signs are told apart
    seen = set()
    for row in logits:
        direction = row[1:] / row[1:].norm()
        errors = [(direction - candidate).norm().item() for candidate in candidates]
        assert min(errors) < 1e-6, errors
        seen.add(errors.index(min(errors)))
    # the rows' own embeddings differ, so a norm that read them would not give one direction
    x0 = w["model.embed_tokens.weight"][torch.tensor(ids)]
    assert (x0[0] / x0[0].norm() - x0[1] / x0[1].norm()).norm() > 0.1


def test_the_second_norm_test_tells_a_parallel_block_apart(monkeypatch):
    """The check above is not empty: with a block whose feed-forward reads the residual as it
    was before attention (x + attn(n1 x) + ffn(n2 x)) the rows' directions scatter."""
    cfg, w = _dominant_attention_model(13)
    ids = [3, 17, 9, 21, 0, 11, 5, 5, 14]
    before = {}
    real_attention, real_feed_forward = plain.attention_block, plain.feed_forward_block

    def attention_block(x, *args):
        before["x"] = x
        return real_attention(x, *args)

    def feed_forward_block(x, *args):
        return real_feed_forward(before["x"], *args)

    monkeypatch.setattr(plain, "attention_block", attention_block)
    monkeypatch.setattr(plain, "feed_forward_block", feed_forward_block)
    logits = plain.forward(w, cfg, ids)
    directions = torch.stack([row[1:] / row[1:].norm() for row in logits])
    spread = (directions[:, None, :] - directions[None, :, :]).norm(dim=-1)
    pairs_apart = ((spread > 0.1) & ((directions[:, None, :] + directions[None, :, :]).norm(dim=-1) > 0.1))
    assert pairs_apart.sum() > len(ids)


def test_single_rows_of_a_one_layer_model_are_the_rows_of_the_whole():
    """The rows-only form that the tests of long contexts use."""
    cfg = dict(CONFIGS["B"], num_hidden_layers=1)
    w = _random_weights(cfg, 31)
    ids = [(7 * i + 3) % cfg["vocab_size"] for i in range(41)]
    whole = plain.forward(w, cfg, ids)
    rows = [0, 1, 17, 39, 40, 17]
    assert torch.allclose(plain.forward(w, cfg, ids, rows=rows), whole[rows], atol=1e-12)
    with pytest.raises(ValueError):
        plain.forward(_random_weights(dict(CONFIGS["B"]), 31), dict(CONFIGS["B"]), ids, rows=[0])
