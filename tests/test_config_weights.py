"""Configuration, registry, safetensors reading and the loader's one error."""
import json

import numpy as np
import pytest
import torch

from conftest import TINY, tensor_shapes, write_folder

import runtime
from runtime.config import (ConfigError, LlamaConfig, architecture_of, config_from_folder, preset, preset_names,
                            register_architecture, unregister_architecture)
from runtime.engine.loading import build_from_config_dict, write_random_model
from runtime.weights import (SafetensorsFile, TensorSpec, WeightError, check_against, load_folder, open_folder,
                             write_safetensors)


def raw(name="a", **over):
    return {"model_type": "llama", "architectures": ["LlamaForCausalLM"], **TINY[name], **over}


def test_config_reads_its_keys():
    c = LlamaConfig.from_dict(raw("c"))
    assert (c.hidden_size, c.num_attention_heads, c.num_key_value_heads, c.head_dim) == (200, 6, 2, 64)
    assert c.rope_theta == 100000.0 and c.rms_norm_eps == 1e-5 and not c.tie_word_embeddings
    d = dict(raw("a")); del d["head_dim"]; del d["num_key_value_heads"]
    c = LlamaConfig.from_dict(d)
    assert c.head_dim == 16 and c.num_key_value_heads == 4  # head_dim = hidden/heads, kv heads default to heads
    assert LlamaConfig.from_dict(raw(eos_token_id=[2, 7])).eos_token_ids == (2, 7)
    assert LlamaConfig.from_dict(LlamaConfig.from_dict(raw("b")).to_dict()) == LlamaConfig.from_dict(raw("b"))


@pytest.mark.parametrize("bad, word", [
    ({"rope_scaling": {"factor": 2}}, "rope_scaling"), ({"attention_bias": True}, "bias"), ({"mlp_bias": True}, "bias"),
    ({"hidden_act": "gelu"}, "silu"), ({"num_key_value_heads": 3}, "multiple"), ({"head_dim": 15}, "head_dim"),
    ({"head_dim": 258}, "head_dim"), ({"vocab_size": 0}, "positive"), ({"model_type": "mistral"}, "llama")])
def test_config_rejections(bad, word):
    with pytest.raises(ConfigError, match=word):
        LlamaConfig.from_dict(raw(**bad))


def test_config_missing_key_is_named():
    d = raw(); del d["intermediate_size"]
    with pytest.raises(ConfigError, match="intermediate_size"):
        LlamaConfig.from_dict(d)


def test_registry_maps_names_to_models():
    assert architecture_of({"architectures": ["LlamaForCausalLM"]}).config_cls is LlamaConfig
    assert architecture_of({"model_type": "llama"}).config_cls is LlamaConfig
    with pytest.raises(ConfigError, match="no registered architecture"):
        architecture_of({"model_type": "unheard-of"})
    with pytest.raises(ConfigError, match="already registered"):
        register_architecture("llama", LlamaConfig, lambda c: None)
    register_architecture("toy-arch", LlamaConfig, lambda c: "built")
    try:
        assert architecture_of({"model_type": "toy-arch"}).build(None) == "built"
    finally:
        unregister_architecture("toy-arch")


def test_presets_are_data_and_build():
    assert {"tiny-a", "tiny-b", "smollm2-135m", "smollm2-1.7b", "llama-3-8b"} <= set(preset_names())
    _, c, model = build_from_config_dict(preset("smollm2-135m"))
    assert (c.num_hidden_layers, c.hidden_size, c.num_attention_heads, c.num_key_value_heads, c.head_dim,
            c.intermediate_size, c.vocab_size, c.rope_theta, c.tie_word_embeddings) == (30, 576, 9, 3, 64, 1536, 49152, 1e5, True)
    n_params = sum(int(np.prod(s.shape)) for s in model.tensor_specs())
    assert n_params == 134_515_008  # 134.5 M parameters with the tied head counted once
    assert len(model.cache_needs()) == 30 and not model.state_needs()


def test_model_declares_exactly_the_checkpoint_names():
    for name in TINY:
        _, _, model = build_from_config_dict(raw(name))
        assert {s.name: tuple(s.shape) for s in model.tensor_specs()} == tensor_shapes(TINY[name])


def test_safetensors_roundtrip_with_the_library(tmp_path):
    from safetensors.torch import save_file, load_file
    tensors = {"m": torch.randn(5, 7).to(torch.bfloat16), "v": torch.arange(6, dtype=torch.float32),
               "i": torch.arange(4, dtype=torch.int64).reshape(2, 2), "h": torch.randn(3).to(torch.float16)}
    save_file(tensors, str(tmp_path / "lib.safetensors"))
    f = SafetensorsFile(tmp_path / "lib.safetensors")
    assert sorted(f.names()) == sorted(tensors)
    for k, t in tensors.items():
        got = f.tensor(k)
        assert got.dtype == t.dtype and torch.equal(got, t)
    write_safetensors(tmp_path / "own.safetensors", tensors)
    back = load_file(str(tmp_path / "own.safetensors"))
    for k, t in tensors.items():
        assert torch.equal(back[k], t)


def test_safetensors_rejects_bad_sizes(tmp_path):
    import struct
    header = json.dumps({"x": {"dtype": "F32", "shape": [4], "data_offsets": [0, 12]}}).encode()
    (tmp_path / "bad.safetensors").write_bytes(struct.pack("<Q", len(header)) + header + b"\0" * 12)
    with pytest.raises(ValueError, match="invalid size"):
        SafetensorsFile(tmp_path / "bad.safetensors")
    header = json.dumps({"x": {"dtype": "F8_E4M3", "shape": [4], "data_offsets": [0, 4]}}).encode()
    (tmp_path / "bad2.safetensors").write_bytes(struct.pack("<Q", len(header)) + header + b"\0" * 4)
    with pytest.raises(ValueError, match="unsupported dtype"):
        SafetensorsFile(tmp_path / "bad2.safetensors")


def test_loader_keeps_dtypes(tmp_path):
    from safetensors.torch import save_file
    save_file({"m": torch.randn(4, 4).to(torch.bfloat16), "f": torch.randn(4), "t": torch.arange(5, dtype=torch.int64)},
              str(tmp_path / "model.safetensors"))
    specs = [TensorSpec("m", (4, 4)), TensorSpec("f", (4,)), TensorSpec("t", (5,), integer=True)]
    got = load_folder(tmp_path, specs, torch.bfloat16, "cpu")
    assert got["m"].dtype == torch.bfloat16     # bfloat16 is kept
    assert got["f"].dtype == torch.float32      # stored in 32 bits: stays so
    assert got["t"].dtype == torch.int32        # integer table
    got = load_folder(tmp_path, specs, torch.float32, "cpu")
    assert got["m"].dtype == torch.float32 and got["t"].dtype == torch.int32


def test_loader_lists_everything_wrong_in_one_error(tmp_path):
    from safetensors.torch import save_file
    c = TINY["a"]
    folder = write_folder(tmp_path / "m", c, 0)
    from safetensors.torch import load_file
    tensors = load_file(str(folder / "model.safetensors"))
    del tensors["model.layers.1.mlp.up_proj.weight"]
    del tensors["model.norm.weight"]
    tensors["model.layers.0.self_attn.rotary_emb.inv_freq"] = torch.zeros(8)
    tensors["lm_head.weight"] = torch.zeros(c["vocab_size"], c["hidden_size"])  # tied model: its copy of the head is ignored
    tensors["model.layers.0.self_attn.k_proj.weight"] = torch.zeros(64, 64)
    save_file(tensors, str(folder / "model.safetensors"))
    _, _, model = build_from_config_dict(raw("a"))
    with pytest.raises(WeightError) as info:
        check_against(model.tensor_specs(), open_folder(folder), model.ignored_tensors())
    text = str(info.value)
    for needle in ("missing (2)", "model.layers.1.mlp.up_proj.weight", "model.norm.weight", "unexpected (1)",
                   "rotary_emb.inv_freq", "wrong shape (1)", "k_proj.weight: file has [64, 64], model expects [32, 64]"):
        assert needle in text, needle
    assert "lm_head.weight" not in text
    _, _, untied = build_from_config_dict(raw("b"))
    assert untied.ignored_tensors() == ()


def test_loader_leaves_extra_tensors_alone(tmp_path, capsys):
    """A tensor the model does not declare is no fault by itself (the reference checks the expected set only,
    runtime/checkpoint.py:44-58): the folder loads, the extra is named on stderr; strict mode refuses it."""
    from safetensors.torch import load_file, save_file
    folder = write_folder(tmp_path / "m", TINY["a"], 0)
    tensors = load_file(str(folder / "model.safetensors"))
    tensors["model.layers.0.self_attn.rotary_emb.inv_freq"] = torch.zeros(8)
    save_file(tensors, str(folder / "model.safetensors"))
    _, _, model = build_from_config_dict(raw("a"))
    got = load_folder(folder, model.tensor_specs(), torch.bfloat16, "cpu", ignored=model.ignored_tensors())
    assert set(got) == {s.name for s in model.tensor_specs()}
    assert "rotary_emb.inv_freq" in capsys.readouterr().err
    assert check_against(model.tensor_specs(), open_folder(folder)) == ["model.layers.0.self_attn.rotary_emb.inv_freq"]
    with pytest.raises(WeightError, match="unexpected \\(1\\)"):
        load_folder(folder, model.tensor_specs(), torch.bfloat16, "cpu", ignored=model.ignored_tensors(), strict=True)


def test_loader_duplicate_across_shards_and_empty_folder(tmp_path):
    from safetensors.torch import save_file
    with pytest.raises(FileNotFoundError):
        open_folder(tmp_path)
    save_file({"x": torch.zeros(2)}, str(tmp_path / "a.safetensors"))
    save_file({"x": torch.zeros(2)}, str(tmp_path / "b.safetensors"))
    with pytest.raises(WeightError, match="appears in"):
        open_folder(tmp_path)


def test_random_weights_mode_writes_a_loadable_folder(tmp_path):
    a = write_random_model(tmp_path / "one", "tiny-b", seed=1)
    b = write_random_model(tmp_path / "two", "tiny-b", seed=1)
    c = write_random_model(tmp_path / "three", "tiny-b", seed=2)
    assert (a / "config.json").exists() and (a / "model.safetensors").exists()
    assert (a / "model.safetensors").read_bytes() == (b / "model.safetensors").read_bytes()
    assert (a / "model.safetensors").read_bytes() != (c / "model.safetensors").read_bytes()
    arch, cfg = config_from_folder(a)
    model = arch.build(cfg)
    check_against(model.tensor_specs(), open_folder(a))
    f = SafetensorsFile(a / "model.safetensors")
    norm = f.tensor("model.norm.weight").float()
    mat = f.tensor("model.layers.0.mlp.up_proj.weight").float()
    assert abs(norm.mean() - 1) < 0.01 and 0.015 < norm.std() < 0.025
    assert abs(mat.mean()) < 1e-3 and 0.019 < mat.std() < 0.021
    assert "lm_head.weight" in f.names()  # tiny-b is untied
