"""Loading by tensor name, precision kept, one error for everything wrong (no GPU)."""
import json

import pytest
import torch
from safetensors.torch import load_file, save_file

from edge_infer_amd import Qwen3Config, WeightsError, write_model_folder
from edge_infer_amd.engine.model import expected_parameters, model_parameters
from edge_infer_amd.weights import match_parameters, read_tensors
from helpers import make_folder, tiny_config


def expected_for(name):
    cfg = tiny_config(name)
    return cfg, expected_parameters(cfg.model_spec(), cfg.checkpoint_name)


def test_random_folder_round_trip(tmp_path):
    folder = make_folder("B", tmp_path)
    cfg, expected = expected_for("B")
    assert Qwen3Config.from_dict(json.loads((folder / "config.json").read_text())) == cfg
    tensors = read_tensors(folder)
    params = match_parameters(expected, tensors)
    assert set(params) == {name for name, (_, spec) in expected.items() if not spec.optional}
    assert all(t.dtype == torch.bfloat16 for t in tensors.values())
    q = params["layers.2.mixer.q_proj.weight"]
    assert tuple(q.shape) == (8 * 32, 96)                 # [out, in] as stored
    assert abs(q.float().std().item() - 0.02) < 0.002     # N(0, 0.02)
    n = params["layers.0.norm1.weight"].float()
    assert 0.9 <= n.min() and n.max() <= 1.1 and n.std() > 0.03   # 1 + U(-0.1, 0.1)
    # the same seed gives the same bytes, another seed does not
    again = write_model_folder(tmp_path / "again", cfg, 1)
    other = write_model_folder(tmp_path / "other", cfg, 2)
    a, b, c = (load_file(str(p / "model.safetensors")) for p in (folder, again, other))
    assert all(torch.equal(a[k], b[k]) for k in a)
    assert not torch.equal(a["lm_head.weight"], c["lm_head.weight"])


def test_tied_head_is_not_stored_and_resolves_to_the_embedding(tmp_path):
    folder = make_folder("A", tmp_path)
    cfg, expected = expected_for("A")
    tensors = read_tensors(folder)
    assert "lm_head.weight" not in tensors
    params = match_parameters(expected, tensors, optional={"head.weight": "embed.weight"})
    assert params["head.weight"] is params["embed.weight"]
    # untied configuration without a head: one clear error
    with pytest.raises(WeightsError, match="lm_head.weight"):
        match_parameters(expected, tensors)
    # an explicit head wins over the tie, also under its alias
    tensors["model.lm_head.weight"] = torch.zeros(256, 64, dtype=torch.bfloat16)
    params = match_parameters(expected, tensors, optional={"head.weight": "embed.weight"},
                              aliases=cfg.checkpoint_aliases)
    assert params["head.weight"] is tensors["model.lm_head.weight"]
    # both names at once: which one is meant cannot be known
    tensors["lm_head.weight"] = torch.ones(256, 64, dtype=torch.bfloat16)
    with pytest.raises(WeightsError, match="stored twice") as caught:
        match_parameters(expected, tensors, optional={"head.weight": "embed.weight"},
                         aliases=cfg.checkpoint_aliases)
    assert caught.value.duplicate == ["lm_head.weight"]


def test_one_error_lists_missing_unexpected_and_wrong_shapes(tmp_path):
    folder = make_folder("B", tmp_path)
    _, expected = expected_for("B")
    tensors = read_tensors(folder)
    del tensors["model.layers.1.mlp.up_proj.weight"]
    del tensors["model.norm.weight"]
    tensors["model.layers.7.self_attn.q_proj.weight"] = torch.zeros(2, 2)
    tensors["model.layers.0.self_attn.q_norm.bias"] = torch.zeros(32)
    tensors["model.layers.0.self_attn.k_proj.weight"] = torch.zeros(96, 32)   # transposed
    with pytest.raises(WeightsError) as info:
        match_parameters(expected, tensors)
    error = info.value
    assert sorted(error.missing) == ["model.layers.1.mlp.up_proj.weight", "model.norm.weight"]
    assert error.unexpected == ["model.layers.0.self_attn.q_norm.bias",
                                "model.layers.7.self_attn.q_proj.weight"]
    assert error.wrong_shape == [("model.layers.0.self_attn.k_proj.weight", (32, 96), (96, 32))]
    text = str(error)
    for piece in ("missing tensors (2)", "unexpected tensors (2)", "wrong shapes (1)",
                  "expected [32, 96] got [96, 32]"):
        assert piece in text


def test_stored_precision_is_kept(tmp_path):
    tensors = {
        "a": torch.randn(4, 4, dtype=torch.float32),
        "b": torch.randn(4, 4).to(torch.bfloat16),
        "c": torch.randn(4, 4).to(torch.float16),
        "d": torch.arange(6, dtype=torch.int64),
        "e": torch.randn(3, dtype=torch.float64),
    }
    (tmp_path / "config.json").write_text("{}")
    save_file(tensors, str(tmp_path / "model.safetensors"))
    loaded = read_tensors(tmp_path)
    assert loaded["a"].dtype == torch.float32 and torch.equal(loaded["a"], tensors["a"])
    assert loaded["b"].dtype == torch.bfloat16
    assert loaded["c"].dtype == torch.bfloat16
    assert loaded["d"].dtype == torch.int32 and loaded["d"].tolist() == list(range(6))
    assert loaded["e"].dtype == torch.float32


def test_sharded_checkpoint_and_path_containment(tmp_path):
    save_file({"x": torch.ones(2)}, str(tmp_path / "part1.safetensors"))
    save_file({"y": torch.zeros(3)}, str(tmp_path / "part2.safetensors"))
    index = {"weight_map": {"x": "part1.safetensors", "y": "part2.safetensors"}}
    (tmp_path / "model.safetensors.index.json").write_text(json.dumps(index))
    loaded = read_tensors(tmp_path)
    assert set(loaded) == {"x", "y"}
    index["weight_map"]["y"] = "../outside.safetensors"
    (tmp_path / "model.safetensors.index.json").write_text(json.dumps(index))
    with pytest.raises(ValueError, match="inside"):
        read_tensors(tmp_path)
    (tmp_path / "model.safetensors.index.json").unlink()
    with pytest.raises(FileNotFoundError):
        read_tensors(tmp_path)


def test_the_container_is_read_by_this_package_and_refuses_what_does_not_add_up(tmp_path):
    """The reader agrees with the library that wrote the file, gives views of the mapping
    (no bytes read until touched) and refuses headers that lie."""
    import struct
    from edge_infer_amd.weights.safetensors_file import SafetensorsFile
    tensors = {"m": torch.arange(12, dtype=torch.float32).reshape(3, 4),
               "h": torch.randn(5, 2).to(torch.float16), "empty": torch.zeros(0, 7),
               "flags": torch.tensor([True, False, True]), "bytes": torch.arange(5, dtype=torch.uint8)}
    path = tmp_path / "model.safetensors"
    save_file(tensors, str(path), metadata={"format": "pt"})
    container = SafetensorsFile(path)
    assert sorted(container.names()) == sorted(tensors) and container.metadata == {"format": "pt"}
    for name, tensor in tensors.items():
        assert container.shape(name) == tuple(tensor.shape) and container.dtype(name) == tensor.dtype
        assert torch.equal(container.tensor(name), tensor)
    loaded = read_tensors(tmp_path)
    assert loaded["flags"].dtype == torch.int32 and loaded["flags"].tolist() == [1, 0, 1]
    assert loaded["bytes"].dtype == torch.int32 and loaded["h"].dtype == torch.bfloat16
    # a view, not a copy: two reads of a tensor share their bytes; writing to it changes no file
    view = container.tensor("m")
    assert view.data_ptr() == container.tensor("m").data_ptr()
    view.fill_(7.0)
    assert torch.equal(SafetensorsFile(path).tensor("m"), tensors["m"])
    raw = path.read_bytes()
    (length,) = struct.unpack("<Q", raw[:8])
    header = json.loads(raw[8:8 + length])

    def rewritten(change):
        changed = json.loads(json.dumps(header))
        change(changed)
        text = json.dumps(changed).encode()
        (tmp_path / "bad.safetensors").write_bytes(struct.pack("<Q", len(text)) + text
                                                    + raw[8 + length:])
        return tmp_path / "bad.safetensors"
    with pytest.raises(ValueError, match="does not fit"):
        SafetensorsFile(rewritten(lambda h: h["m"].update(shape=[3, 5])))
    with pytest.raises(ValueError, match="does not fit"):
        SafetensorsFile(rewritten(lambda h: h["m"].update(data_offsets=[0, 10 ** 9])))
    with pytest.raises(ValueError, match="unsupported"):
        SafetensorsFile(rewritten(lambda h: h["m"].update(dtype="F8_E4M3")))
    (tmp_path / "bad.safetensors").write_bytes(struct.pack("<Q", 10 ** 12) + b"{}")
    with pytest.raises(ValueError, match="header claims"):
        SafetensorsFile(tmp_path / "bad.safetensors")
    (tmp_path / "bad.safetensors").write_bytes(b"abc")
    with pytest.raises(ValueError, match="too short"):
        SafetensorsFile(tmp_path / "bad.safetensors")
    # an index that names a tensor its file does not hold
    (tmp_path / "model.safetensors.index.json").write_text(
        json.dumps({"weight_map": {"nowhere": "model.safetensors"}}))
    with pytest.raises(ValueError, match="hold it"):
        read_tensors(tmp_path)


def test_parameter_inventory_matches_the_architecture():
    cfg = tiny_config("B")
    every = model_parameters(cfg.model_spec())
    params = {name: p for name, p in every.items() if not p.optional}
    per_layer = 11   # 2 norms, q k v o, q_norm k_norm, gate up down
    assert len(params) == 3 + per_layer * cfg.num_hidden_layers
    # optional: a bias for each of the seven projections of a layer and for the head
    assert len(every) - len(params) == 7 * cfg.num_hidden_layers + 1
    total = sum(torch.Size(p.shape).numel() for p in params.values())
    H, V, I, Q, KV, d = 96, 381, 200, 256, 32, 32
    layer = 2 * H + Q * H + 2 * KV * H + H * Q + 2 * d + 3 * I * H
    assert total == 2 * V * H + H + 3 * layer


def test_verbose_listing_of_what_is_read(tmp_path, monkeypatch, capsys):
    """EDGE_INFER_VERBOSE_WEIGHTS=1 lists every tensor with its file, shape and type (the
    reference's loader has such a listing too, frontend/checkpoint.py:88-99); without it
    nothing is printed."""
    folder = make_folder("A", tmp_path)
    read_tensors(folder)
    assert capsys.readouterr().out == ""
    monkeypatch.setenv("EDGE_INFER_VERBOSE_WEIGHTS", "1")
    tensors = read_tensors(folder)
    lines = capsys.readouterr().out.strip().split("\n")
    assert len(lines) == len(tensors)
    assert "model.safetensors: model.embed_tokens.weight [256, 64] bfloat16" in lines


def test_optional_biases_are_taken_when_the_checkpoint_holds_them(tmp_path):
    """runtime/include/models/qwen3_model.hpp:371-403: each projection and the head may have
    a bias; none is required, a wrong shape is an error, and `model.lm_head.bias` is an
    alias (bindings/python/include/decoder_weight_mapper.hpp:114-121)."""
    cfg, expected = expected_for("B")
    assert cfg.checkpoint_name("layers.1.mixer.k_proj.bias") == \
        "model.layers.1.self_attn.k_proj.bias"
    assert cfg.checkpoint_name("layers.0.ffn.down_proj.bias") == "model.layers.0.mlp.down_proj.bias"
    assert cfg.checkpoint_name("head.bias") == "lm_head.bias"
    with pytest.raises(KeyError):
        cfg.checkpoint_name("layers.0.norm1.bias")
    plain = read_tensors(make_folder("B", tmp_path))
    assert not any(name.endswith(".bias") for name in plain)
    folder = write_model_folder(tmp_path / "biased", cfg, 1, biases=True)
    tensors = read_tensors(folder)
    # the weights are the ones the same seed gives without biases?  No: the draws interleave;
    # what is fixed is that every optional tensor is there with its shape
    params = match_parameters(expected, tensors)
    assert set(params) == set(expected)
    assert tuple(params["layers.2.mixer.q_proj.bias"].shape) == (8 * 32,)
    assert tuple(params["layers.2.ffn.gate_proj.bias"].shape) == (200,)
    assert tuple(params["head.bias"].shape) == (381,)
    # some biases only: fine
    some = {name: t for name, t in tensors.items()
            if not name.endswith(".bias") or "q_proj" in name}
    assert "layers.0.mixer.v_proj.bias" not in match_parameters(expected, some)
    # the alias of the head's bias
    some["model.lm_head.bias"] = tensors["lm_head.bias"]
    params = match_parameters(expected, some, aliases=cfg.checkpoint_aliases)
    assert params["head.bias"] is tensors["lm_head.bias"]
    # a wrong shape and a bias the model has no use for are reported
    tensors["model.layers.0.self_attn.o_proj.bias"] = torch.zeros(95, dtype=torch.bfloat16)
    tensors["model.layers.0.input_layernorm.bias"] = torch.zeros(96, dtype=torch.bfloat16)
    with pytest.raises(WeightsError) as caught:
        match_parameters(expected, tensors)
    assert caught.value.wrong_shape == [("model.layers.0.self_attn.o_proj.bias", (96,), (95,))]
    assert caught.value.unexpected == ["model.layers.0.input_layernorm.bias"]
    assert not caught.value.missing
