"""A plain, slow Qwen3-dense implementation used only as the oracle of the tests.

Whole sequences, no cache, one function per part, float64 arithmetic on the CPU
(rotation angles are formed in float32 exactly as the reference forms them and
then evaluated in float64).  Nothing here imports the product package: formulas
are written from the reference's text and every function cites the lines it
follows.  Paths are relative to the reference checkout.
"""
from __future__ import annotations

import json
import math
from pathlib import Path

import numpy as np
import torch

F64 = torch.float64


# ----------------------------------------------------------------------------
# parts
# ----------------------------------------------------------------------------
def embedding(ids, table):
    """x0[r, :] = E[id[r], :], no scaling.

    operators/src/cuda/execution.cu:67-78 (gather_rows_kernel),
    runtime/src/qwen3.cpp:296.
    """
    ids = torch.as_tensor(ids, dtype=torch.long)
    return table.to(F64)[ids]


def rms_norm(x, weight, eps):
    """y_j = x_j / sqrt(mean(x^2) + eps) * w_j; the weight multiplies directly.

    operators/include/operators/core/cpu_reference.hpp:48-64,
    operators/src/cuda/rms_norm_cuda.cu:74 (rsqrt(sum / n + eps)).
    """
    x = x.to(F64)
    mean_square = (x * x).sum(dim=-1, keepdim=True) / x.shape[-1]
    return x / torch.sqrt(mean_square + eps) * weight.to(F64)


def linear(x, weight_out_in, bias=None):
    """y = x . W^T for a checkpoint matrix stored [out, in].

    operators/src/cuda/execution.cu:299-324 (m=out, n=rows, k=in, OP_T on the
    [out, in] bytes), bindings/python/include/decoder_weight_mapper.hpp:166-174.
    """
    y = x.to(F64) @ weight_out_in.to(F64).T
    if bias is not None:
        y = y + bias.to(F64)
    return y


def rope_angles(positions, head_dim, theta):
    """angle[p, i] = float(p) * (1 / pow(theta, 2i / d)), all in float32.

    runtime/include/models/qwen3_model.hpp:418-424: `std::pow(float, float)`, the C
    library's single-precision power, whose result is the double-precision power rounded
    once to float32; it is formed that way here, so that no other library's last bit of a
    float32 power enters the angle.
    """
    half = head_dim // 2
    i = np.arange(half, dtype=np.float32)
    exponent = (np.float32(2.0) * i) / np.float32(head_dim)
    power = np.power(np.float64(np.float32(theta)), exponent.astype(np.float64))
    frequency = np.float32(1.0) / power.astype(np.float32)
    pos = np.asarray(positions, dtype=np.int64).astype(np.float32)
    angle = (pos[:, None] * frequency[None, :]).astype(np.float32)
    return torch.from_numpy(angle.astype(np.float64))


def rope(x, positions, theta):
    """Rotate-half on [rows, heads, d]: pairs (i, i + d/2);
    x' = x cos a - y sin a, y' = x sin a + y cos a.

    operators/src/cuda/execution.cu:79-122 (rotate_kernel, float branch
    :118-121), runtime/src/qwen.cpp:319-333.
    """
    x = x.to(F64)
    rows, heads, d = x.shape
    half = d // 2
    angle = rope_angles(positions, d, theta)  # [rows, half]
    cos = torch.cos(angle)[:, None, :]
    sin = torch.sin(angle)[:, None, :]
    first, second = x[..., :half], x[..., half:]
    return torch.cat([first * cos - second * sin, first * sin + second * cos], dim=-1)


def attention(q, k, v, positions=None, window=None, key_positions=None):
    """Causal grouped-query attention of one sequence.

    q [S, nq, d], k and v [S, nkv, d]; query head h reads kv head
    h // (nq // nkv); scores scaled by 1/sqrt(d); key t is visible to the query
    at absolute position p iff t <= p (and t > p - window when a window is
    given; the reference has no window).  Softmax over visible keys.
    `key_positions`: where the keys sit when q holds only some rows of the sequence
    (then `positions` are those rows' places); by default the queries' own places.

    operators/src/cuda/execution.cu:137-179 (attention_scalar_kernel),
    runtime/src/qwen.cpp:374-402.
    """
    q, k, v = q.to(F64), k.to(F64), v.to(F64)
    S, nq, d = q.shape
    nkv = k.shape[1]
    group = nq // nkv
    if positions is None:
        positions = torch.arange(S)
    positions = torch.as_tensor(positions, dtype=torch.long)
    out = torch.zeros(S, nq, d, dtype=F64)
    scale = 1.0 / math.sqrt(d)
    # keys of a whole sequence sit at the same positions as its queries
    key_pos = positions if key_positions is None else torch.as_tensor(key_positions, dtype=torch.long)
    for h in range(nq):
        g = h // group
        scores = (q[:, h, :] @ k[:, g, :].T) * scale  # [S, S]
        visible = key_pos[None, :] <= positions[:, None]
        if window is not None:
            visible &= key_pos[None, :] > positions[:, None] - window
        scores = scores.masked_fill(~visible, float("-inf"))
        m = scores.max(dim=-1, keepdim=True).values
        w = torch.exp(scores - m)
        out[:, h, :] = (w @ v[:, g, :]) / w.sum(dim=-1, keepdim=True)
    return out


def silu(x):
    """silu(z) = z / (1 + exp(-z)).

    operators/include/operators/core/cpu_reference.hpp:37-44,
    operators/src/cuda/silu_cuda.cu:11-32.
    """
    x = x.to(F64)
    return x / (1.0 + torch.exp(-x))


def swiglu(gate, up):
    """silu(gate) * up.  operators/src/cuda/silu_cuda.cu:44-56,
    runtime/include/execution/decoder.hpp:162-165."""
    return silu(gate) * up.to(F64)


# ----------------------------------------------------------------------------
# block and model
# ----------------------------------------------------------------------------
def attention_block(x, w, cfg, layer, positions, rows=None):
    """RMSNorm -> q/k/v -> per-head q/k RMSNorm -> RoPE -> attention -> o.

    runtime/include/execution/decoder.hpp:121-158; the per-head norm comes
    before the rotation (:125-136) and uses the model's one eps.  Each projection takes
    a bias when the checkpoint holds one (runtime/include/models/qwen3_model.hpp:386-395).
    `rows`: the output for these rows of x only (keys and values of every row are still
    made); what makes sequences of tens of thousands of tokens affordable.
    """
    p = f"model.layers.{layer}."
    S = x.shape[0]
    nq, nkv, d = cfg["num_attention_heads"], cfg["num_key_value_heads"], head_dim_of(cfg)
    h = rms_norm(x, w[p + "input_layernorm.weight"], cfg["rms_norm_eps"])
    def project(name, heads):
        return linear(h, w[p + f"self_attn.{name}.weight"],
                      w.get(p + f"self_attn.{name}.bias")).reshape(S, heads, d)

    q, k, v = project("q_proj", nq), project("k_proj", nkv), project("v_proj", nkv)
    q = rms_norm(q, w[p + "self_attn.q_norm.weight"], cfg["rms_norm_eps"])
    k = rms_norm(k, w[p + "self_attn.k_norm.weight"], cfg["rms_norm_eps"])
    q = rope(q, positions, cfg["rope_theta"])
    k = rope(k, positions, cfg["rope_theta"])
    if rows is None:
        a = attention(q, k, v, positions)
    else:
        rows = torch.as_tensor(rows, dtype=torch.long)
        a = attention(q[rows], k, v, torch.as_tensor(positions, dtype=torch.long)[rows],
                      key_positions=positions)
    return linear(a.reshape(a.shape[0], nq * d), w[p + "self_attn.o_proj.weight"],
                  w.get(p + "self_attn.o_proj.bias"))


def feed_forward_block(x, w, cfg, layer):
    """RMSNorm -> gate, up -> silu(gate) * up -> down.
    runtime/include/execution/decoder.hpp:161-166; optional biases
    runtime/include/models/qwen3_model.hpp:396-403."""
    p = f"model.layers.{layer}."
    h = rms_norm(x, w[p + "post_attention_layernorm.weight"], cfg["rms_norm_eps"])
    g = linear(h, w[p + "mlp.gate_proj.weight"], w.get(p + "mlp.gate_proj.bias"))
    u = linear(h, w[p + "mlp.up_proj.weight"], w.get(p + "mlp.up_proj.bias"))
    return linear(swiglu(g, u), w[p + "mlp.down_proj.weight"], w.get(p + "mlp.down_proj.bias"))


def head_dim_of(cfg):
    """runtime/include/models/qwen3_model.hpp:166-174."""
    if "head_dim" in cfg:
        return cfg["head_dim"]
    return cfg["hidden_size"] // cfg["num_attention_heads"]


def head_weight(w, cfg):
    """lm_head.weight, or the embedding when tie_word_embeddings is True.
    bindings/python/include/decoder_weight_mapper.hpp:81-102."""
    if "lm_head.weight" in w:
        return w["lm_head.weight"]
    if cfg.get("tie_word_embeddings", False) is True:
        return w["model.embed_tokens.weight"]
    raise KeyError("lm_head.weight")


def forward(w, cfg, ids, positions=None, rows=None):
    """Logits [S, V] (float64) of one whole sequence.

    runtime/include/execution/decoder.hpp:119-169, runtime/src/qwen3.cpp:293-299.
    `rows` (models of one layer only, whose rows need nothing of each other beyond the
    layer's keys and values): logits [len(rows), V] at these places.
    """
    S = len(ids)
    if positions is None:
        positions = list(range(S))
    x = embedding(ids, w["model.embed_tokens.weight"])
    if rows is not None and cfg["num_hidden_layers"] != 1:
        raise ValueError("single rows can be asked of a model of one layer only")
    for layer in range(cfg["num_hidden_layers"]):
        if rows is None:
            x = x + attention_block(x, w, cfg, layer, positions)
        else:
            x = x[torch.as_tensor(rows, dtype=torch.long)] \
                + attention_block(x, w, cfg, layer, positions, rows=rows)
        x = x + feed_forward_block(x, w, cfg, layer)
    y = rms_norm(x, w["model.norm.weight"], cfg["rms_norm_eps"])
    return linear(y, head_weight(w, cfg), w.get("lm_head.bias"))   # qwen3_model.hpp:371-372


# ----------------------------------------------------------------------------
# sampling
# ----------------------------------------------------------------------------
_M64 = (1 << 64) - 1


def uniform(seed, stream, counter):
    """The framework's documented counter-based draw in (0, 1]: splitmix64's
    finalizer of seed + golden * (stream * 2^32 + counter + 1); the top 24 bits
    plus one, times 2^-24.  (The reference draws from one cuRAND state seeded by
    the wall clock, runtime/src/inference.cpp:272-274, which no test can pin.)"""
    z = (seed + 0x9E3779B97F4A7C15 * (((stream << 32) + counter + 1) & _M64)) & _M64
    z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & _M64
    z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & _M64
    z ^= z >> 31
    return ((z >> 40) + 1) * (1.0 / 16777216.0)


def filtered_distribution(logits, temperature, top_p, top_k):
    """(order, probabilities of the kept prefix) in float32 as the reference's
    kernel computes them.

    operators/src/cuda/execution.cu:193-234: z = logit / T (NaN -> -inf), sort
    descending (ties: lowest index first, runtime/src/qwen.cpp:467-470),
    k = min(top_k, V), e_i = exp(z_i - z_0), keep the shortest prefix whose mass
    reaches top_p * total, at least one element and including the one that
    crosses.
    """
    z = np.asarray(logits, dtype=np.float32).copy()
    z[np.isnan(z)] = -np.inf
    greedy = temperature <= 0 or min(top_k, len(z)) == 1
    if not greedy:
        z = (z / np.float32(temperature)).astype(np.float32)
    order = np.lexsort((np.arange(len(z)), -z.astype(np.float64)))
    if greedy or not np.isfinite(z[order[0]]):
        return order[:1], np.ones(1, dtype=np.float32)
    k = min(top_k, len(z))
    e = np.exp((z[order[:k]] - z[order[0]]).astype(np.float32)).astype(np.float32)
    total = np.float32(0)
    for value in e:
        total = np.float32(total + value)
    threshold = np.float32(np.float32(top_p) * total)
    retained = np.float32(0)
    count = 0
    while True:
        retained = np.float32(retained + e[count])
        count += 1
        if not (count < k and retained < threshold):
            break
    return order[:count], (e[:count] / retained).astype(np.float32)


def sample(logits, temperature, top_p, top_k, u):
    """Token drawn with the uniform number u in (0, 1]: the first kept element
    whose cumulative mass reaches u * retained.
    operators/src/cuda/execution.cu:223-231."""
    order, prob = filtered_distribution(logits, temperature, top_p, top_k)
    if len(order) == 1:
        return int(order[0])
    # work on unnormalised masses exactly as the kernel does
    z = np.asarray(logits, dtype=np.float32).copy()
    z[np.isnan(z)] = -np.inf
    z = (z / np.float32(temperature)).astype(np.float32)
    e = np.exp((z[order] - z[order[0]]).astype(np.float32)).astype(np.float32)
    retained = np.float32(0)
    for value in e:
        retained = np.float32(retained + value)
    target = np.float32(np.float32(u) * retained)
    cumulative = np.float32(0)
    for i, value in enumerate(e):
        cumulative = np.float32(cumulative + value)
        if cumulative >= target:
            return int(order[i])
    return int(order[-1])


def generate(w, cfg, prompt, max_length, temperature=0.0, top_p=1.0, top_k=1, seed=0,
             stream=0, stop_ids=None):
    """Tokens generated after `prompt`, recomputing the whole sequence each step.

    runtime/src/inference.cpp:367-418: max_length counts prompt plus generated
    tokens; a stop token ends the request and is not returned.
    """
    if stop_ids is None:
        stop_ids = {cfg["eos_token_id"]}
    ids = list(prompt)
    out = []
    limit = max_length
    if limit <= len(ids):
        return out
    step = 0
    while True:
        logits = forward(w, cfg, ids)[-1].to(torch.float32).numpy()
        token = sample(logits, temperature, top_p, top_k, uniform(seed, stream, step))
        step += 1
        if token in stop_ids:
            break
        out.append(token)
        ids.append(token)
        if len(ids) >= limit:
            break
    return out


# ----------------------------------------------------------------------------
# reading a model folder without the product's loader
# ----------------------------------------------------------------------------
def read_folder(path):
    """(config dict, {name: float64 tensor}) from config.json + model.safetensors."""
    from safetensors import safe_open

    path = Path(path)
    cfg = json.loads((path / "config.json").read_text())
    weights = {}
    with safe_open(str(path / "model.safetensors"), framework="pt", device="cpu") as f:
        for name in f.keys():
            weights[name] = f.get_tensor(name).to(F64)
    return cfg, weights
