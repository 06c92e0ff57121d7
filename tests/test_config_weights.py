"""Configuration, registry and weight-file errors (CPU)."""
import copy
import json
import os

import pytest
import torch

from conftest import TINY_A, TINY_B
from kv_cache_optimization_for_llm_amd.config.model_config import ConfigError, LlamaConfig, read_config_json
from kv_cache_optimization_for_llm_amd.config.registry import (ARCHITECTURES, RegistryError,
                                                               architecture_for)
from kv_cache_optimization_for_llm_amd.models.builder import spec_for_config, tensor_specs_for_config
from kv_cache_optimization_for_llm_amd.weights.loader import (WeightError, checkpoint_index,
                                                              target_dtype, validate)
from kv_cache_optimization_for_llm_amd.weights.random_init import write_random_model


def test_config_reads_every_key():
    c = LlamaConfig.from_dict(TINY_B)
    assert (c.vocab_size, c.hidden_size, c.intermediate_size, c.num_hidden_layers) == (384, 96, 256, 3)
    assert (c.num_attention_heads, c.num_key_value_heads, c.head_dim) == (4, 1, 24)
    assert c.rms_norm_eps == 1e-6 and c.rope_theta == 500000.0 and not c.tie_word_embeddings
    assert c.rope_scaling.factor == 8.0 and c.rope_scaling.original_max_position_embeddings == 64
    assert c.eos_token_id == (382, 383)
    a = LlamaConfig.from_dict(TINY_A)
    assert a.rope_scaling is None and a.tie_word_embeddings and a.eos_token_id == (255,)


def test_config_defaults_follow_the_keys():
    d = {k: v for k, v in TINY_A.items() if k not in ("head_dim", "num_key_value_heads")}
    c = LlamaConfig.from_dict(d)
    assert c.head_dim == 64 // 4 and c.num_key_value_heads == 4


@pytest.mark.parametrize("patch, word", [
    ({"num_key_value_heads": 3}, "multiple"),
    ({"head_dim": 15}, "even"),
    ({"head_dim": 18}, "multiples of 4"),
    ({"head_dim": 260}, "above 256"),
    ({"hidden_act": "gelu"}, "hidden_act"),
    ({"attention_bias": True}, "attention_bias"),
    ({"mlp_bias": True}, "mlp_bias"),
    ({"rope_scaling": {"rope_type": "yarn", "factor": 2.0}}, "rope_type"),
    ({"rope_scaling": {"rope_type": "llama3", "factor": 2.0}}, "low_freq_factor"),
    ({"vocab_size": None}, "vocab_size"),
    ({"rms_norm_eps": None}, "rms_norm_eps"),
    ({"torch_dtype": "float16"}, "torch_dtype"),
])
def test_config_errors_name_the_key(patch, word):
    d = copy.deepcopy(TINY_A)
    d.update(patch)
    with pytest.raises(ConfigError) as e:
        LlamaConfig.from_dict(d)
    assert word in str(e.value)


def test_hidden_not_multiple_of_heads_needs_head_dim():
    d = dict(TINY_A, hidden_size=66)
    d.pop("head_dim")
    with pytest.raises(ConfigError):
        LlamaConfig.from_dict(d)
    assert LlamaConfig.from_dict(dict(d, head_dim=16)).head_dim == 16


def test_registry_picks_by_architecture_name():
    assert architecture_for(TINY_A).name == "LlamaForCausalLM"
    with pytest.raises(RegistryError) as e:
        architecture_for(dict(TINY_A, architectures=["NoSuchModel"]))
    assert "LlamaForCausalLM" in str(e.value) and "NoSuchModel" in str(e.value)
    with pytest.raises(RegistryError):
        architecture_for({k: v for k, v in TINY_A.items() if k != "architectures"})


def test_spec_is_data_layer_by_layer():
    cfg, spec = spec_for_config(TINY_B)
    assert len(spec.layers) == 3 and [c.layer for c in spec.order] == [0, 1, 2]
    m = spec.layers[1].mixer
    assert m.kind == "gqa_attention" and m.params["num_kv_heads"] == 1 and m.params["head_dim"] == 24
    assert m.params["position"].kind == "rotary" and m.params["position"].params["theta"] == 500000.0
    # the frequency rule is a named parameter of the part, its constants beside it
    assert m.params["position"].params["frequencies"] == "llama3"
    assert m.params["position"].params["frequency_params"] == dict(
        factor=8.0, low_freq_factor=1.0, high_freq_factor=4.0, original_max_position_embeddings=64)
    assert spec_for_config(TINY_A)[1].layers[0].mixer.params["position"].params["frequencies"] == "plain"
    assert spec.layers[2].feed_forward.params["intermediate_size"] == 256
    assert spec.head_name == "lm_head.weight"
    assert spec_for_config(TINY_A)[1].head_name is None


def test_random_model_folder_roundtrip(tmp_path):
    d = write_random_model(str(tmp_path / "m"), TINY_A, seed=3)
    assert read_config_json(d)["hidden_size"] == 64
    idx = checkpoint_index(d)
    specs = tensor_specs_for_config(TINY_A)
    assert set(idx) == set(specs)
    validate(idx, specs)
    from safetensors.torch import load_file
    w = load_file(os.path.join(d, "model.safetensors"))
    assert all(t.dtype == torch.bfloat16 for t in w.values())
    e = w["model.embed_tokens.weight"].float()
    assert abs(e.std().item() - 0.02) < 0.002 and abs(e.mean().item()) < 0.002
    n = w["model.norm.weight"].float()
    # 1 + U(-0.1, 0.1), rounded to bfloat16 (spacing 2^-8 below 1, 2^-7 above)
    assert 0.9 - 2 ** -8 <= n.min().item() and n.max().item() <= 1.1 + 2 ** -7 and n.std().item() > 0.02
    # same seed -> same values, whatever else is in the model; another seed -> other values
    d2 = write_random_model(str(tmp_path / "m2"), dict(TINY_A, num_hidden_layers=1), seed=3)
    w2 = load_file(os.path.join(d2, "model.safetensors"))
    assert torch.equal(w2["model.layers.0.mlp.up_proj.weight"], w["model.layers.0.mlp.up_proj.weight"])
    d3 = write_random_model(str(tmp_path / "m3"), TINY_A, seed=4)
    assert not torch.equal(load_file(os.path.join(d3, "model.safetensors"))["model.norm.weight"],
                           w["model.norm.weight"])


def test_one_error_lists_missing_unexpected_and_misshapen(tmp_path):
    from safetensors.torch import load_file, save_file
    d = write_random_model(str(tmp_path / "m"), TINY_B, seed=1)
    path = os.path.join(d, "model.safetensors")
    w = load_file(path)
    del w["model.layers.1.mlp.down_proj.weight"]
    del w["lm_head.weight"]
    w["model.layers.0.self_attn.q_norm.weight"] = torch.ones(24, dtype=torch.bfloat16)
    w["model.layers.2.self_attn.k_proj.weight"] = torch.zeros(48, 96, dtype=torch.bfloat16)
    w["model.norm.weight"] = torch.ones(96, dtype=torch.int32)
    save_file(w, path)
    with pytest.raises(WeightError) as e:
        validate(checkpoint_index(d), tensor_specs_for_config(TINY_B))
    msg = str(e.value)
    assert "missing tensors (2)" in msg and "model.layers.1.mlp.down_proj.weight" in msg and "lm_head.weight" in msg
    assert "unexpected tensors (1)" in msg and "q_norm" in msg
    assert "wrong shapes (1)" in msg and "[48, 96]" in msg and "[24, 96]" in msg
    assert "unsupported dtypes (1)" in msg and "I32" in msg


def test_tied_model_may_carry_an_unused_head(tmp_path):
    from safetensors.torch import load_file, save_file
    d = write_random_model(str(tmp_path / "m"), TINY_A, seed=1)
    path = os.path.join(d, "model.safetensors")
    w = load_file(path)
    w["lm_head.weight"] = w["model.embed_tokens.weight"].clone()
    save_file(w, path)
    _, spec = spec_for_config(TINY_A)
    validate(checkpoint_index(d), tensor_specs_for_config(TINY_A), spec.ignorable_tensors)


def test_a_checkpoint_in_shards_is_read_through_its_index(tmp_path):
    """Larger checkpoints come as several files and ``model.safetensors.index.json`` naming, per
    tensor, the file that holds it (the reference reads the one-file form only,
    ``base/src/model.cu:15-84``): the same tensors come out of the shards as out of one file, a
    tensor that no shard holds is reported by name, and so is a shard the index names that is
    not there."""
    from safetensors.torch import load_file, save_file
    from kv_cache_optimization_for_llm_amd.weights.loader import load_tensors
    whole = write_random_model(str(tmp_path / "whole"), TINY_B, seed=9)
    w = load_file(os.path.join(whole, "model.safetensors"))
    names = sorted(w)
    shards = {"model-00001-of-00002.safetensors": names[: len(names) // 3],
              "model-00002-of-00002.safetensors": names[len(names) // 3:]}
    d = tmp_path / "sharded"
    d.mkdir()
    (d / "config.json").write_text(json.dumps(TINY_B))
    for fname, part in shards.items():
        save_file({n: w[n] for n in part}, str(d / fname))
    index = {"metadata": {"total_size": 0}, "weight_map": {n: f for f, part in shards.items() for n in part}}
    (d / "model.safetensors.index.json").write_text(json.dumps(index))
    specs = tensor_specs_for_config(TINY_B)
    got = load_tensors(str(d), specs, torch.bfloat16, "cpu")
    want = load_tensors(whole, specs, torch.bfloat16, "cpu")
    assert sorted(got) == sorted(want) == sorted(specs)
    assert all(torch.equal(got[n], want[n]) and got[n].dtype == want[n].dtype for n in want)
    assert {os.path.basename(f) for f, _ in checkpoint_index(str(d)).values()} == set(shards)
    # a tensor that is in no shard
    lost = names[-1]
    save_file({n: w[n] for n in shards["model-00002-of-00002.safetensors"] if n != lost},
              str(d / "model-00002-of-00002.safetensors"))
    with pytest.raises(WeightError) as e:
        load_tensors(str(d), specs, torch.bfloat16, "cpu")
    assert "missing tensors (1)" in str(e.value) and lost in str(e.value)
    # a shard that the index names and the folder does not hold
    os.remove(d / "model-00001-of-00002.safetensors")
    with pytest.raises(WeightError) as e:
        checkpoint_index(str(d))
    assert "model-00001-of-00002.safetensors" in str(e.value)


def test_broken_files_are_refused(tmp_path):
    d = tmp_path / "m"
    d.mkdir()
    (d / "config.json").write_text(json.dumps(TINY_A))
    with pytest.raises(WeightError):
        checkpoint_index(str(d))
    (d / "model.safetensors").write_bytes(b"\x10\x00")
    with pytest.raises(WeightError):
        checkpoint_index(str(d))
    (d / "model.safetensors").write_bytes((10 ** 9).to_bytes(8, "little") + b"{}")
    with pytest.raises(WeightError):
        checkpoint_index(str(d))
    hdr = json.dumps({"t": {"dtype": "F32", "shape": [4], "data_offsets": [0, 16]}}).encode()
    (d / "model.safetensors").write_bytes(len(hdr).to_bytes(8, "little") + hdr + b"\0" * 8)
    with pytest.raises(WeightError) as e:
        checkpoint_index(str(d))
    assert "outside the file" in str(e.value)


def test_dtype_rule():
    bf, f32 = torch.bfloat16, torch.float32
    assert target_dtype(bf, "matrix", bf) == bf          # kept in bfloat16
    assert target_dtype(bf, "matrix", f32) == f32        # widened exactly for the 32-bit path
    assert target_dtype(f32, "vector", bf) == f32        # stored in 32-bit stays so
    # float16 does not fit into bfloat16: it is widened to 32-bit on either engine
    assert target_dtype(torch.float16, "matrix", bf) == f32 and target_dtype(torch.float16, "matrix", f32) == f32
    assert target_dtype(torch.int64, "table", bf) == torch.int32


def test_random_weights_command_writes_the_same_folder_as_the_function(tmp_path):
    from kv_cache_optimization_for_llm_amd.weights import random_init
    cfg_file = tmp_path / "c.json"
    cfg_file.write_text(json.dumps(TINY_B))
    assert random_init.main(["--config", str(cfg_file), "--out", str(tmp_path / "cmd"), "--seed", "5"]) == 0
    write_random_model(str(tmp_path / "fn"), TINY_B, 5)
    a = (tmp_path / "cmd" / "model.safetensors").read_bytes()
    b = (tmp_path / "fn" / "model.safetensors").read_bytes()
    assert a == b and read_config_json(str(tmp_path / "cmd")) == read_config_json(str(tmp_path / "fn"))
