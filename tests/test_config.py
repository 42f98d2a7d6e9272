"""Typed configuration and the architecture registry (no GPU)."""
import json

import pytest

from edge_infer_amd import Qwen3Config
from edge_infer_amd.config import (ConfigError, known_architectures, read_config,
                                   register_architecture, resolve_architecture,
                                   unregister_architecture)
from edge_infer_amd.config.specs import ModelSpec, ScheduleEntry
from helpers import tiny_config


def raw(name, **extra):
    d = tiny_config(name).to_dict()
    d.update(extra)
    return d


@pytest.mark.parametrize("name", ["A", "B"])
def test_round_trip(name):
    cfg = tiny_config(name)
    assert Qwen3Config.from_dict(cfg.to_dict()) == cfg
    spec = cfg.model_spec()
    assert len(spec.layers) == cfg.num_hidden_layers == len(spec.schedule)
    mixer = spec.layers[0].mixer
    assert (mixer.n_heads, mixer.n_kv_heads, mixer.head_dim) == (
        cfg.num_attention_heads, cfg.num_key_value_heads, cfg.head_dim)
    assert mixer.qk_norm and mixer.window is None
    assert mixer.position.theta == cfg.rope_theta and mixer.qk_norm_eps == cfg.rms_norm_eps
    assert spec.layers[0].feed_forward.intermediate_size == cfg.intermediate_size
    assert spec.final_norm.eps == cfg.rms_norm_eps


def test_head_dim_default_and_divisibility():
    d = raw("A")
    del d["head_dim"]
    assert Qwen3Config.from_dict(d).head_dim == 64 // 4
    d["hidden_size"] = 66
    with pytest.raises(ConfigError, match="divisible"):
        Qwen3Config.from_dict(d)


@pytest.mark.parametrize("key", ["vocab_size", "hidden_size", "num_hidden_layers",
                                 "num_attention_heads", "num_key_value_heads",
                                 "intermediate_size", "max_position_embeddings", "bos_token_id",
                                 "eos_token_id", "rms_norm_eps", "rope_theta"])
def test_required_keys(key):
    d = raw("B")
    del d[key]
    with pytest.raises(ConfigError, match=key):
        Qwen3Config.from_dict(d)


@pytest.mark.parametrize("extra, message", [
    ({"hidden_act": "gelu"}, "SiLU"),
    ({"rope_scaling": {"type": "yarn", "factor": 4}}, "rotary"),
    ({"use_sliding_window": True, "sliding_window": 128}, "sliding"),
    ({"sliding_window": 128}, "sliding"),
    ({"layer_types": ["full_attention", "sliding_attention"]}, "full-attention"),
    ({"tie_word_embeddings": 1}, "boolean"),
    ({"num_key_value_heads": 3}, "multiple"),
    ({"head_dim": 15}, "even"),
    ({"rms_norm_eps": 0.0}, "rms_norm_eps"),
    ({"vocab_size": 2.5}, "vocab_size"),
    ({"eos_token_id": [1, 2]}, "eos_token_id"),
])
def test_refusals(extra, message):
    with pytest.raises(ConfigError, match=message):
        Qwen3Config.from_dict(raw("A", **extra))


def test_admitted_variants():
    Qwen3Config.from_dict(raw("A", rope_scaling=None))
    Qwen3Config.from_dict(raw("A", rope_scaling={}))
    Qwen3Config.from_dict(raw("A", use_sliding_window=False, sliding_window=4096))
    Qwen3Config.from_dict(raw("A", layer_types=["full_attention"] * 2, hidden_act="silu"))


def test_registry(tmp_path):
    assert "Qwen3ForCausalLM" in known_architectures()
    assert resolve_architecture({"architectures": ["Qwen3ForCausalLM"]}).config_class is Qwen3Config
    assert resolve_architecture({"model_type": "qwen3"}).config_class is Qwen3Config
    with pytest.raises(KeyError, match="Qwen3ForCausalLM"):
        resolve_architecture({"architectures": ["SomethingElse"]})
    with pytest.raises(ValueError, match="already"):
        register_architecture("Qwen3ForCausalLM", Qwen3Config)

    class Other:
        @classmethod
        def from_dict(cls, d):
            return cls()
    register_architecture("ToyForCausalLM", Other, model_types=("toy",))
    try:
        (tmp_path / "config.json").write_text(json.dumps({"architectures": ["ToyForCausalLM"]}))
        entry, cfg, _ = read_config(tmp_path)
        assert entry.name == "ToyForCausalLM" and isinstance(cfg, Other)
    finally:
        unregister_architecture("ToyForCausalLM")
    with pytest.raises(KeyError):
        resolve_architecture({"model_type": "toy"})


def test_schedule_validation():
    spec = tiny_config("A").model_spec()
    def with_schedule(schedule):
        return ModelSpec(**{**spec.__dict__, "schedule": tuple(schedule)})
    # a layer may run twice, and a layer may read another's cache
    with_schedule([ScheduleEntry(0, 0), ScheduleEntry(1, 1), ScheduleEntry(0, 2),
                   ScheduleEntry(1, 1, writes_cache=False)]).validate()
    with pytest.raises(ValueError, match="two writers"):
        with_schedule([ScheduleEntry(0, 0), ScheduleEntry(1, 0)]).validate()
    with pytest.raises(ValueError, match="before it is written"):
        with_schedule([ScheduleEntry(0, 1, writes_cache=False), ScheduleEntry(1, 1)]).validate()
    with pytest.raises(ValueError, match="names layer"):
        with_schedule([ScheduleEntry(5, 0)]).validate()


def test_checkpoint_names():
    name = Qwen3Config.checkpoint_name
    assert name("embed.weight") == "model.embed_tokens.weight"
    assert name("layers.3.mixer.q_norm.weight") == "model.layers.3.self_attn.q_norm.weight"
    assert name("layers.0.ffn.down_proj.weight") == "model.layers.0.mlp.down_proj.weight"
    assert name("layers.12.norm2.weight") == "model.layers.12.post_attention_layernorm.weight"
    assert name("head.weight") == "lm_head.weight"
    with pytest.raises(KeyError):
        name("layers.0.mixer.gate.weight")


def test_a_model_names_the_kernel_libraries_it_will_run():
    """What is compiled at a model's first use is what that model needs: head sizes 64 and 128
    in bfloat16 take the matrix-core attention library, everything else the generic one, and a
    part that says nothing (a toy part of a test) asks for nothing."""
    import torch
    from edge_infer_amd import Qwen3Config
    from edge_infer_amd.engine.model import DecoderModel
    from edge_infer_amd.parts import register_mixer, unregister
    from helpers import TINY_A

    small = Qwen3Config(**TINY_A).model_spec()                       # head_dim 16
    wide = Qwen3Config(**{**TINY_A, "head_dim": 128}).model_spec()
    assert set(DecoderModel.kernel_libraries(small, torch.float32)) == \
        {"rowwise", "gemm_f32", "rope_store", "attention_generic"}
    assert set(DecoderModel.kernel_libraries(small, torch.bfloat16)) == \
        {"rowwise", "gemm_bf16", "rope_store", "attention_generic"}
    assert set(DecoderModel.kernel_libraries(wide, torch.bfloat16)) == \
        {"rowwise", "gemm_bf16", "rope_store", "attention_mfma"}
    assert "attention_mfma" not in DecoderModel.kernel_libraries(wide, torch.float32)

    class Silent:            # no kernel_libraries
        pass
    register_mixer("toy_silent", Silent)
    try:
        import dataclasses
        layer = dataclasses.replace(small.layers[0],
                                    mixer=dataclasses.replace(small.layers[0].mixer, kind="toy_silent"))
        toy = dataclasses.replace(small, layers=(layer,) * len(small.layers))
        assert "attention_generic" not in DecoderModel.kernel_libraries(toy, torch.float32)
    finally:
        unregister("mixer", "toy_silent")
