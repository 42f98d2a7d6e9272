"""Shared test fixtures: two tiny Qwen3 configurations that differ in every size and
option, and tolerances that are fixed here once."""
from pathlib import Path

import torch

# float32 engine against the float64 plain implementation, relative to the largest logit
# (the largest seen in the whole suite is 4.7e-6, on a layer of the 8B widths)
F32_REL = 2e-5
# bfloat16 engine against the plain implementation: root-mean-square and maximum error
# relative to the root-mean-square and the maximum logit (bfloat16 keeps 8 significant
# bits, 2^-9 relative per rounding; a few dozen roundings accumulate per token).  The largest
# seen: 0.6 % / 0.75 % on the tiny models, 0.86 % / 0.91 % on a layer of the 8B widths.
BF16_RMS_REL = 1.2e-2
BF16_MAX_REL = 1.5e-2
# the same for the tests of thousands of tokens with raised q/k norm weights, whose scores
# (and with them the rounding of bfloat16 queries and keys) are more than twice as large:
# 1.46 % / 2.03 % seen
BF16_LONG_RMS_REL = 2e-2
BF16_LONG_MAX_REL = 3e-2

TINY_A = dict(vocab_size=256, hidden_size=64, num_hidden_layers=2, num_attention_heads=4,
              num_key_value_heads=2, head_dim=16, intermediate_size=128,
              max_position_embeddings=128, bos_token_id=0, eos_token_id=255, rms_norm_eps=1e-6,
              rope_theta=10000.0, tie_word_embeddings=True)
TINY_B = dict(vocab_size=381, hidden_size=96, num_hidden_layers=3, num_attention_heads=8,
              num_key_value_heads=1, head_dim=32, intermediate_size=200,
              max_position_embeddings=256, bos_token_id=1, eos_token_id=380, rms_norm_eps=1e-5,
              rope_theta=1000000.0, tie_word_embeddings=False)
# head size 128 (the matrix-core attention kernels in bfloat16), for contexts of thousands of
# tokens; `max_position_embeddings` may be raised by the caller
LONG = dict(vocab_size=1003, hidden_size=256, num_hidden_layers=2, num_attention_heads=8,
            num_key_value_heads=4, head_dim=128, intermediate_size=640,
            max_position_embeddings=5120, bos_token_id=0, eos_token_id=1, rms_norm_eps=1e-6,
            rope_theta=1000000.0, tie_word_embeddings=False)
SEEDS = {"A": 0, "B": 1}
CONFIGS = {"A": TINY_A, "B": TINY_B}


def tiny_config(name):
    from edge_infer_amd import Qwen3Config
    return Qwen3Config(**CONFIGS[name])


def make_folder(name, root):
    from edge_infer_amd import write_model_folder
    path = Path(root) / f"tiny_{name}"
    if not (path / "model.safetensors").is_file():
        write_model_folder(path, tiny_config(name), SEEDS[name])
    return path


def make_long_folder(root, seed=3, head_norm_scale=1.5, **overrides):
    """A model folder of the `LONG` shape whose q/k norm weights are raised by
    `head_norm_scale`: that more than doubles the scores, so attention is peaked, and a key
    that is left out, read twice or read from a foreign page moves the logits by far more
    than the tolerance."""
    from safetensors.torch import load_file, save_file
    from edge_infer_amd import Qwen3Config, write_model_folder
    path = Path(root) / "long_model"
    write_model_folder(path, Qwen3Config(**dict(LONG, **overrides)), seed=seed)
    tensors = load_file(str(path / "model.safetensors"))
    for name in tensors:
        if name.endswith("q_norm.weight") or name.endswith("k_norm.weight"):
            tensors[name] = (tensors[name].float() * head_norm_scale).to(torch.bfloat16)
    save_file(tensors, str(path / "model.safetensors"))
    return path


def random_ids(vocab, count, seed):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, vocab, (count,), generator=g).tolist()


_SEEN = {}


def _record(kind, value, what):
    import os
    path = os.environ.get("EI_TEST_RECORD_ERRORS")
    if path and value > _SEEN.get(kind, (0.0, ""))[0]:
        _SEEN[kind] = (value, what)
        with open(path, "a") as out:
            out.write(f"{kind} {value:.3e} {what}\n")


def assert_close_f32(actual, expected, what=""):
    actual, expected = actual.double().cpu(), expected.double().cpu()
    scale = expected.abs().max().item()
    err = (actual - expected).abs().max().item()
    _record("f32", err / scale, what)
    assert err <= F32_REL * scale, f"{what}: max error {err:.3e} against scale {scale:.3e}"


def assert_close_bf16(actual, expected, what="", rms_rel=BF16_RMS_REL, max_rel=BF16_MAX_REL):
    actual, expected = actual.double().cpu(), expected.double().cpu()
    diff = actual - expected
    rms = diff.pow(2).mean().sqrt().item()
    ref_rms = expected.pow(2).mean().sqrt().item()
    worst = diff.abs().max().item()
    scale = expected.abs().max().item()
    _record("bf16_rms", rms / ref_rms, what)
    _record("bf16_max", worst / scale, what)
    assert rms <= rms_rel * ref_rms, f"{what}: rms error {rms:.3e} against {ref_rms:.3e}"
    assert worst <= max_rel * scale, f"{what}: max error {worst:.3e} against {scale:.3e}"


def assert_close(dtype, actual, expected, what="", **bf16_bounds):
    if dtype == "float32":
        assert_close_f32(actual, expected, what)
    else:
        assert_close_bf16(actual, expected, what, **bf16_bounds)


def assert_close_long(dtype, actual, expected, what=""):
    """For the long-context models with raised q/k norm weights."""
    assert_close(dtype, actual, expected, what, rms_rel=BF16_LONG_RMS_REL,
                 max_rel=BF16_LONG_MAX_REL)
