"""Weights by name: round trip, one error for every misfit, dtypes, the random-weights mode."""
import os

import pytest
import torch

from tiny_configs import TINY
from tokenizer_amd.config import Qwen2Config
from tokenizer_amd.models.qwen2 import qwen2_spec
from tokenizer_amd.parts import TensorSpec, expected_tensors
from tokenizer_amd.weights import (SafetensorsFile, WeightError, load_weights, random_tensors, save_safetensors,
                                   write_random_model)


def expected(name="A"):
    return expected_tensors(qwen2_spec(Qwen2Config.from_dict(TINY[name][0])))


def test_random_model_folder_round_trips(tmp_path):
    cfg = Qwen2Config.from_dict(TINY["B"][0])
    folder = write_random_model(cfg, 2, str(tmp_path / "m"))
    assert sorted(os.listdir(folder)) == ["config.json", "model.safetensors"]
    source = SafetensorsFile(os.path.join(folder, "model.safetensors"))
    assert set(source.names()) == set(expected("B"))
    assert all(source.info(n)[1] == torch.bfloat16 for n in source.names())
    again = random_tensors(expected("B"), 2)
    for name in source.names():
        assert torch.equal(source.tensor(name), again[name])
    # Readable by the safetensors package too (the plain implementation reads folders with it).
    from safetensors.torch import load_file
    other = load_file(os.path.join(folder, "model.safetensors"))
    assert torch.equal(other["model.norm.weight"], torch.ones(96, dtype=torch.bfloat16))
    w = other["model.layers.1.mlp.up_proj.weight"].float()
    assert w.shape == (272, 96) and abs(float(w.std()) - 0.02) < 0.002 and abs(float(w.mean())) < 0.002
    assert float(other["model.layers.0.self_attn.q_proj.bias"].float().abs().max()) > 0


def test_seed_and_name_fix_each_tensor():
    spec = {"x.weight": TensorSpec((8, 8)), "y.weight": TensorSpec((8, 8))}
    one = random_tensors(spec, 7)
    assert not torch.equal(one["x.weight"], one["y.weight"])
    assert torch.equal(one["x.weight"], random_tensors({"x.weight": TensorSpec((8, 8))}, 7)["x.weight"])
    assert not torch.equal(one["x.weight"], random_tensors(spec, 8)["x.weight"])


def test_dtypes_are_kept_as_the_rules_say(tmp_path):
    tensors = random_tensors(expected(), 0)
    tensors["model.norm.weight"] = torch.ones(64, dtype=torch.float32) * 1.0000001
    path = str(tmp_path / "model.safetensors")
    save_safetensors(path, tensors)
    bf = load_weights(path, expected(), torch.bfloat16)
    assert bf["model.layers.0.mlp.up_proj.weight"].dtype == torch.bfloat16
    assert bf["model.norm.weight"].dtype == torch.float32          # small vectors are float32
    assert float(bf["model.norm.weight"][0]) == float(torch.tensor(1.0000001, dtype=torch.float32))
    assert bf["model.layers.0.self_attn.q_proj.bias"].dtype == torch.float32
    f32 = load_weights(path, expected(), torch.float32)
    assert f32["model.layers.0.mlp.up_proj.weight"].dtype == torch.float32
    assert torch.equal(f32["model.layers.0.mlp.up_proj.weight"], bf["model.layers.0.mlp.up_proj.weight"].float())
    # "keep" leaves a 32-bit tensor in 32 bits and an integer table becomes int32.
    extra = {"a": TensorSpec((2,), role="keep"), "t": TensorSpec((3,), role="table")}
    save_safetensors(path, {"a": torch.tensor([1.5, 2.5]), "t": torch.tensor([1, 2, 3], dtype=torch.int64)})
    out = load_weights(path, extra, torch.bfloat16)
    assert out["a"].dtype == torch.float32 and out["t"].dtype == torch.int32 and out["t"].tolist() == [1, 2, 3]


def test_one_error_lists_missing_unexpected_and_wrong_shapes(tmp_path):
    tensors = random_tensors(expected(), 0)
    del tensors["model.layers.1.self_attn.k_proj.bias"]
    del tensors["model.norm.weight"]
    tensors["lm_head.weight"] = torch.zeros(256, 64, dtype=torch.bfloat16)
    tensors["model.layers.0.mlp.gate_proj.weight"] = torch.zeros(64, 128, dtype=torch.bfloat16)
    tensors["model.layers.0.input_layernorm.weight"] = torch.zeros(64, dtype=torch.int32)
    path = str(tmp_path / "model.safetensors")
    save_safetensors(path, tensors)
    with pytest.raises(WeightError) as err:
        load_weights(path, expected(), torch.bfloat16)
    e = err.value
    assert e.missing == ["model.layers.1.self_attn.k_proj.bias", "model.norm.weight"]
    assert e.unexpected == ["lm_head.weight"]
    assert e.wrong_shape == [("model.layers.0.mlp.gate_proj.weight", (64, 128), (128, 64))]
    assert e.wrong_dtype == [("model.layers.0.input_layernorm.weight", torch.int32)]
    text = str(e)
    for word in ("missing (2)", "unexpected (1)", "wrong shape (1)", "is [64, 128], wanted [128, 64]", "lm_head.weight"):
        assert word in text


def test_tensors_the_model_does_not_read_are_a_warning_alone(tmp_path):
    # A tied model saved with a redundant head, an export with rotary buffers: the reference takes what it asks
    # for by name and never looks at the rest (qwen-infer/src/model.rs:776-786).
    from tokenizer_amd.weights import UnexpectedTensors
    tensors = random_tensors(expected(), 0)
    tensors["lm_head.weight"] = tensors["model.embed_tokens.weight"].clone()
    tensors["model.layers.0.self_attn.rotary_emb.inv_freq"] = torch.ones(8)
    path = str(tmp_path / "model.safetensors")
    save_safetensors(path, tensors)
    with pytest.warns(UnexpectedTensors, match="lm_head.weight") as caught:
        out = load_weights(path, expected(), torch.bfloat16)
    ours = [str(w.message) for w in caught if isinstance(w.message, UnexpectedTensors)]
    assert len(ours) == 1 and "rotary_emb.inv_freq" in ours[0] and set(out) == set(expected())
    with pytest.raises(WeightError) as err:
        load_weights(path, expected(), torch.bfloat16, strict=True)
    assert err.value.unexpected == ["lm_head.weight", "model.layers.0.self_attn.rotary_emb.inv_freq"]
    assert not err.value.missing


def test_a_model_in_shards_beside_an_index(tmp_path):
    import json
    tensors = random_tensors(expected("B"), 2)
    names = sorted(tensors)
    shards = {"model-00001-of-00002.safetensors": names[::2], "model-00002-of-00002.safetensors": names[1::2]}
    for file_name, held in shards.items():
        save_safetensors(str(tmp_path / file_name), {n: tensors[n] for n in held})
    index = {"metadata": {}, "weight_map": {n: f for f, held in shards.items() for n in held}}
    (tmp_path / "model.safetensors.index.json").write_text(json.dumps(index))
    out = load_weights(str(tmp_path), expected("B"), torch.bfloat16)
    assert set(out) == set(names) and all(torch.equal(out[n].float(), tensors[n].float()) for n in names)
    # A tensor the index promises but its shard does not hold is missing; a shard that is not there says so.
    save_safetensors(str(tmp_path / "model-00002-of-00002.safetensors"), {n: tensors[n] for n in names[1::2][1:]})
    with pytest.raises(WeightError) as err:
        load_weights(str(tmp_path), expected("B"), torch.bfloat16)
    assert err.value.missing == [names[1]]
    (tmp_path / "model-00001-of-00002.safetensors").unlink()
    with pytest.raises(WeightError, match="no weight file"):
        load_weights(str(tmp_path), expected("B"), torch.bfloat16)


def test_untied_model_needs_its_head(tmp_path):
    tensors = random_tensors(expected("B"), 2)
    del tensors["lm_head.weight"]
    path = str(tmp_path / "model.safetensors")
    save_safetensors(path, tensors)
    with pytest.raises(WeightError) as err:
        load_weights(path, expected("B"), torch.float32)
    assert err.value.missing == ["lm_head.weight"]


def test_truncated_and_absent_files(tmp_path):
    path = str(tmp_path / "model.safetensors")
    save_safetensors(path, random_tensors(expected(), 0))
    data = open(path, "rb").read()
    open(path, "wb").write(data[:len(data) // 2])
    with pytest.raises(WeightError) as err:
        load_weights(path, expected(), torch.float32)
    assert "truncated" in str(err.value)
    with pytest.raises(WeightError) as err:
        load_weights(str(tmp_path / "nothing"), expected(), torch.float32)
    assert "no weight file" in str(err.value)
