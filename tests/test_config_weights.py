"""Configuration, registry, safetensors and weight errors (no GPU)."""

from __future__ import annotations

import json

import pytest
import torch

from conftest import TINY_A, TINY_B
from paged_llm_rs_amd.config import GenerationConfig, Qwen3Config, architectures, load_config
from paged_llm_rs_amd.errors import ConfigError, UnsupportedError, WeightError
from paged_llm_rs_amd.parts.model import declare_parameters
from paged_llm_rs_amd.weights import (ParamDecl, SafetensorsFile, check_declared, load_weights,
                                      write_random_model, write_safetensors)


def qwen3_06b() -> dict:
    """The published Qwen3-0.6B config (reference: config.rs:236-254)."""
    return {
        "model_type": "qwen3", "hidden_act": "silu", "attention_bias": False, "sliding_window": None,
        "hidden_size": 1024, "intermediate_size": 3072, "num_hidden_layers": 28,
        "num_attention_heads": 16, "num_key_value_heads": 8, "head_dim": 128, "rms_norm_eps": 1e-6,
        "rope_theta": 1000000.0, "vocab_size": 151936, "max_position_embeddings": 40960,
        "tie_word_embeddings": True,
    }


def test_published_config_parses_and_its_widths_follow():
    """config.rs:262-270"""
    c = load_config(qwen3_06b())
    assert isinstance(c, Qwen3Config)
    assert c.kv_group_size == 2 and c.query_width == 2048 and c.kv_width == 1024
    assert c.query_width != c.hidden_size


@pytest.mark.parametrize("field,value", [
    ("model_type", "llama"), ("hidden_act", "gelu"), ("attention_bias", True), ("sliding_window", 4096),
    ("rope_scaling", {"type": "yarn", "factor": 4.0}), ("num_key_value_heads", 5),
])
def test_a_field_the_engine_would_ignore_is_refused(field, value):
    """config.rs:272-323"""
    d = qwen3_06b()
    d[field] = value
    with pytest.raises(UnsupportedError):
        load_config(d)


def test_rotary_base_in_either_layout_and_scaled_tables_refused():
    """config.rs:289-316"""
    assert load_config(qwen3_06b()).rope_theta == 1e6
    nested = qwen3_06b()
    del nested["rope_theta"]
    nested["rope_parameters"] = {"rope_theta": 1000000.0, "rope_type": "default"}
    assert load_config(nested).rope_theta == 1e6
    neither = qwen3_06b()
    del neither["rope_theta"]
    with pytest.raises(ConfigError):
        load_config(neither)
    nested["rope_parameters"]["rope_type"] = "yarn"
    with pytest.raises(UnsupportedError):
        load_config(nested)


def test_missing_keys_and_bad_values_are_config_errors():
    d = qwen3_06b()
    del d["head_dim"]
    with pytest.raises(ConfigError, match="head_dim"):
        load_config(d)
    d = qwen3_06b()
    d["hidden_size"] = -3
    with pytest.raises(ConfigError):
        load_config(d)


def test_registry_chooses_by_architecture_then_model_type():
    assert "Qwen3ForCausalLM" in architectures()
    d = qwen3_06b()
    d["architectures"] = ["Qwen3ForCausalLM"]
    assert isinstance(load_config(d), Qwen3Config)
    d["architectures"] = ["MambaForCausalLM"]
    with pytest.raises(UnsupportedError, match="MambaForCausalLM"):
        load_config(d)
    d = qwen3_06b()
    d["model_type"] = "gpt2"
    with pytest.raises(UnsupportedError):
        load_config(d)


def test_model_spec_has_no_size_of_its_own():
    for cfg in (TINY_A, TINY_B):
        spec = load_config(cfg).model_spec()
        assert len(spec.layers) == cfg["num_hidden_layers"] == len(spec.schedule)
        m = spec.layers[0].mixer
        assert (m.num_heads, m.num_kv_heads, m.head_dim) == (
            cfg["num_attention_heads"], cfg["num_key_value_heads"], cfg["head_dim"])
        assert spec.layers[0].feed_forward.intermediate_size == cfg["intermediate_size"]
        assert spec.layers[0].norm.eps == cfg["rms_norm_eps"]
        assert m.position.max_positions == cfg["max_position_embeddings"]


def test_generation_config(tmp_path):
    """config.rs:185-231"""
    (tmp_path / "config.json").write_text(json.dumps({"eos_token_id": 7}))
    g = GenerationConfig.from_dir(tmp_path)
    assert g.eos_token_ids == [7] and g.temperature is None
    (tmp_path / "generation_config.json").write_text(json.dumps(
        {"eos_token_id": [151645, 151643], "temperature": 0.6, "top_p": 0.95, "top_k": 20}))
    g = GenerationConfig.from_dir(tmp_path)
    assert g.eos_token_ids == [151645, 151643]
    assert abs(g.temperature - 0.6) < 1e-9 and abs(g.top_p - 0.95) < 1e-9 and g.top_k == 20
    (tmp_path / "generation_config.json").write_text(json.dumps({"top_k": 0}))
    assert GenerationConfig.from_dir(tmp_path).top_k is None


# --- safetensors and weights ----------------------------------------------------------------

def test_own_reader_agrees_with_the_library_reader(tmp_path):
    from safetensors.torch import load_file, save_file

    tensors = {"a": torch.randn(3, 5), "b": torch.randn(7).to(torch.bfloat16),
               "c": torch.arange(6, dtype=torch.int64).reshape(2, 3)}
    save_file(tensors, str(tmp_path / "lib.safetensors"))
    f = SafetensorsFile(tmp_path / "lib.safetensors")
    assert sorted(f.names()) == ["a", "b", "c"]
    for k, v in tensors.items():
        assert torch.equal(f.tensor(k), v)
    write_safetensors(tmp_path / "own.safetensors", tensors)
    back = load_file(str(tmp_path / "own.safetensors"))
    for k, v in tensors.items():
        assert torch.equal(back[k], v)


def test_random_model_is_seeded_and_complete(tmp_path):
    a = write_random_model(tmp_path / "a", TINY_A, seed=0, std=0.02, gain_std=0.1, dtype="float32")
    b = write_random_model(tmp_path / "b", TINY_A, seed=0, std=0.02, gain_std=0.1, dtype="float32")
    c = write_random_model(tmp_path / "c", TINY_A, seed=1, std=0.02, gain_std=0.1, dtype="float32")
    fa, fb, fc = (SafetensorsFile(p / "model.safetensors") for p in (a, b, c))
    assert json.loads((a / "config.json").read_text())["hidden_size"] == 64
    assert "lm_head.weight" not in fa.names()            # tied
    assert len(fa.names()) == 1 + 2 * 11 + 1
    name = "model.layers.1.self_attn.q_proj.weight"
    assert torch.equal(fa.tensor(name), fb.tensor(name))
    assert not torch.equal(fa.tensor(name), fc.tensor(name))
    assert abs(fa.tensor(name).std().item() - 0.02) < 0.004
    gain = fa.tensor("model.layers.0.input_layernorm.weight")
    assert abs(gain.mean().item() - 1.0) < 0.1 and gain.std().item() > 0.03
    untied = write_random_model(tmp_path / "d", TINY_B, seed=1, dtype="bfloat16")
    fd = SafetensorsFile(untied / "model.safetensors")
    assert fd.shape("lm_head.weight") == (384, 96) and fd.dtype("lm_head.weight") == torch.bfloat16
    assert fd.shape("model.layers.2.self_attn.q_proj.weight") == (192, 96)   # head_dim is its own field


def test_weight_errors_list_missing_unexpected_and_wrong_shapes(tmp_path):
    """One error with everything in it (the reference reports one tensor at a time:
    weights.rs:51-66, tests/forward.rs:81-92)."""
    d = write_random_model(tmp_path / "m", TINY_B, seed=1, dtype="float32")
    f = SafetensorsFile(d / "model.safetensors")
    tensors = {n: f.tensor(n).clone() for n in f.names()}
    del tensors["model.layers.1.mlp.up_proj.weight"]
    del tensors["model.norm.weight"]
    tensors["model.layers.0.self_attn.rotary_emb.inv_freq"] = torch.zeros(16)
    tensors["model.layers.2.self_attn.k_norm.weight"] = torch.zeros(96)
    write_safetensors(d / "model.safetensors", tensors)
    spec = load_config(d).model_spec()
    with pytest.raises(WeightError) as e:
        load_weights(d, declare_parameters(spec), torch.float32, "cpu")
    text = str(e.value)
    assert "missing (2)" in text and "model.layers.1.mlp.up_proj.weight" in text and "model.norm.weight" in text
    assert "unexpected (1)" in text and "rotary_emb.inv_freq" in text
    assert "wrong shape (1)" in text and "model.layers.2.self_attn.k_norm.weight has shape [96], expected [32]" in text


def test_checkpoint_of_another_shape_is_refused(tmp_path):
    """tests/forward.rs:81-92: one more query head than the checkpoint has."""
    d = write_random_model(tmp_path / "m", TINY_A, seed=0, dtype="float32")
    cfg = dict(TINY_A)
    cfg["num_attention_heads"] += 2
    spec = load_config(cfg).model_spec()
    with pytest.raises(WeightError, match="q_proj"):
        load_weights(d, declare_parameters(spec), torch.float32, "cpu")


def test_untied_without_head_is_refused(tmp_path):
    """model/mod.rs:230-234"""
    d = write_random_model(tmp_path / "m", TINY_B, seed=1, dtype="float32")
    f = SafetensorsFile(d / "model.safetensors")
    tensors = {n: f.tensor(n).clone() for n in f.names() if n != "lm_head.weight"}
    write_safetensors(d / "model.safetensors", tensors)
    from paged_llm_rs_amd.parts.model import DecoderModel

    spec = load_config(d).model_spec()
    params = load_weights(d, declare_parameters(spec), torch.float32, "cpu")
    with pytest.raises(WeightError, match="lm_head"):
        DecoderModel(spec, params, torch.float32, "cpu")


def test_resident_dtypes(tmp_path):
    """bfloat16 keeps 16-bit tensors and 32-bit vectors; float32 widens everything."""
    d = write_random_model(tmp_path / "m", TINY_A, seed=0, dtype="bfloat16")
    f = SafetensorsFile(d / "model.safetensors")
    tensors = {n: f.tensor(n).clone() for n in f.names()}
    tensors["model.norm.weight"] = tensors["model.norm.weight"].float()
    write_safetensors(d / "model.safetensors", tensors)
    spec = load_config(d).model_spec()
    w = load_weights(d, declare_parameters(spec), torch.bfloat16, "cpu")
    assert w["model.norm.weight"].dtype == torch.float32
    assert w["model.embed_tokens.weight"].dtype == torch.bfloat16
    w = load_weights(d, declare_parameters(spec), torch.float32, "cpu")
    assert all(t.dtype == torch.float32 for t in w.values())


def test_check_declared_passes_optional():
    decls = [ParamDecl("a", (2, 3)), ParamDecl("b", (4,), "gain", optional=True)]
    check_declared(decls, {"a": (2, 3)}, "x")
    check_declared(decls, {"a": (2, 3), "b": (4,)}, "x")
    with pytest.raises(WeightError):
        check_declared(decls, {"b": (4,)}, "x")
