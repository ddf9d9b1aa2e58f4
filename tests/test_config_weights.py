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


def test_values_of_the_wrong_kind_are_config_errors(tmp_path):
    """Whatever stands where a key's value should (a list for a name, a number for the rotary base's object, a
    file that holds no object, a file cut short), the configuration is refused with one of the engine's own
    errors and nothing else; the generation defaults of such a folder are none."""
    import random

    from paged_llm_rs_amd.errors import PagedLLMError

    for key, value in [("model_type", [1, 2]), ("model_type", {"a": 1}), ("rope_parameters", 5), ("rope_parameters", "x"),
                       ("architectures", [["Qwen3ForCausalLM"]]), ("architectures", [7])]:
        d = qwen3_06b()
        d[key] = value
        with pytest.raises(PagedLLMError):
            load_config(d)
    (tmp_path / "config.json").write_text("[1, 2]")
    with pytest.raises(ConfigError):
        load_config(tmp_path)
    (tmp_path / "generation_config.json").write_text("[3]")
    assert GenerationConfig.from_dir(tmp_path) == GenerationConfig()

    rng = random.Random(0)
    values = [None, 0, -1, 1.5, "x", [], {}, True, 1 << 40, [1, 2], {"rope_theta": "a"}, 1e308, ""]
    for _ in range(500):
        d = qwen3_06b()
        d["architectures"] = ["Qwen3ForCausalLM"]
        for _ in range(rng.randrange(1, 3)):
            key = rng.choice(list(d) + ["rope_parameters", "rope_scaling", "layer_types", "eos_token_id"])
            if rng.random() < 0.2:
                d.pop(key, None)
            else:
                d[key] = rng.choice(values)
        text = json.dumps(d)
        (tmp_path / "config.json").write_text(text[:rng.randrange(len(text))] if rng.random() < 0.1 else text)
        try:
            load_config(tmp_path)
        except PagedLLMError:
            pass
        GenerationConfig.from_dir(tmp_path)


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


def test_the_command_line_says_what_is_wrong_with_its_arguments(tmp_path, capsys):
    """Prompts that are no numbers and files that are not there end the command line with one line and the
    status 1, before anything is loaded (cli.py; the reference's main.rs reports its errors the same way)."""
    from paged_llm_rs_amd.cli import main

    for args, says in [(["--prompt-ids", "a,b"], "token ids are whole numbers"),
                       (["--prompt-ids", "[1,[2]]"], "token ids are whole numbers"),
                       (["--prompt-file", str(tmp_path / "none.txt")], "--prompt-file"),
                       (["--random-weights", str(tmp_path / "none.json")], "--random-weights"),
                       (["--chunk", "some", "--prompt-ids", "1"], "--chunk")]:
        assert main(["--model", str(tmp_path / "model")] + args) == 1
        assert says in capsys.readouterr().err
    (tmp_path / "cut.json").write_text('{"hidden_size": ')
    assert main(["--model", str(tmp_path / "model"), "--random-weights", str(tmp_path / "cut.json")]) == 1
    assert "is not JSON" in capsys.readouterr().err


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


def test_a_damaged_weight_file_is_a_weight_error_and_nothing_else(tmp_path):
    """A header that is cut, is no object, or describes a tensor wrongly (no offsets, a negative or broken shape,
    bytes that do not match the shape or lie outside the file) is refused as a wrong weight file: whatever is
    done to the header's bytes, the reader either reads what the library reader reads or raises WeightError."""
    import random
    import struct

    good = {"a": torch.randn(3, 5), "b": torch.arange(6, dtype=torch.int32)}
    write_safetensors(tmp_path / "good.safetensors", good)
    raw = (tmp_path / "good.safetensors").read_bytes()
    (length,) = struct.unpack("<Q", raw[:8])
    header, data = json.loads(raw[8:8 + length]), raw[8 + length:]

    def rewritten(head) -> bytes:
        blob = json.dumps(head).encode()
        return struct.pack("<Q", len(blob)) + blob + data

    entry = dict(header["a"])
    cases = {
        "no object": rewritten([1, 2]),
        "no entry": rewritten({"a": 5}),
        "no offsets": rewritten({"a": {k: v for k, v in entry.items() if k != "data_offsets"}}),
        "no shape": rewritten({"a": {k: v for k, v in entry.items() if k != "shape"}}),
        "a negative size": rewritten({"a": {**entry, "shape": [-3, -5]}}),
        "a broken size": rewritten({"a": {**entry, "shape": [3.0, "5"]}}),
        "offsets backwards": rewritten({"a": {**entry, "data_offsets": [60, 0]}}),
        "a negative offset": rewritten({"a": {**entry, "data_offsets": [-60, 0]}}),
        "bytes past the end": rewritten({"a": {**entry, "data_offsets": [1 << 40, (1 << 40) + 60]}}),
        "too few bytes": rewritten({"a": {**entry, "data_offsets": [0, 56]}}),
        "an unknown dtype": rewritten({"a": {**entry, "dtype": "F8_E4M3"}}),
        "a dtype that is no name": rewritten({"a": {**entry, "dtype": 32}}),
        "a cut file": raw[:8 + length + 10],
        "a cut header": raw[:8 + length // 2],
        "a header longer than the file": struct.pack("<Q", 1 << 50) + raw[8:],
        "four bytes": raw[:4],
    }
    for what, blob in cases.items():
        (tmp_path / "bad.safetensors").write_bytes(blob)
        with pytest.raises(WeightError):
            SafetensorsFile(tmp_path / "bad.safetensors")
            raise AssertionError(f"{what} was read")

    rng = random.Random(0)
    read, refused = 0, 0
    for _ in range(300):                                     # bytes of the header overwritten at random
        blob = bytearray(raw)
        for _ in range(rng.randrange(1, 4)):
            blob[rng.randrange(0, 8 + length)] = rng.choice(b'0123456789[]{}",:-eE \\x00\xff')
        (tmp_path / "bad.safetensors").write_bytes(bytes(blob))
        try:
            f = SafetensorsFile(tmp_path / "bad.safetensors")
            for name in f.names():
                assert f.tensor(name).numel() == f.tensor(name).reshape(-1).shape[0]
            read += 1
        except WeightError:
            refused += 1
    assert read + refused == 300 and refused > 100


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


# ---- sharded checkpoints -------------------------------------------------------------------------------

def shard_folder(tmp_path, config, seed, pieces=2, dtype="float32"):
    """A model folder whose tensors lie in ``pieces`` files behind model.safetensors.index.json,
    beside the same model in one file; returns (sharded folder, whole folder, shard names)."""
    whole = write_random_model(tmp_path / "whole", config, seed=seed, dtype=dtype)
    f = SafetensorsFile(whole / "model.safetensors")
    names = f.names()
    sharded = tmp_path / "sharded"
    sharded.mkdir()
    (sharded / "config.json").write_text((whole / "config.json").read_text())
    weight_map, shards = {}, []
    for i in range(pieces):
        shard = f"model-{i + 1:05d}-of-{pieces:05d}.safetensors"
        mine = names[i::pieces]                   # interleaved, so neighbouring tensors lie in different files
        write_safetensors(sharded / shard, {n: f.tensor(n).clone() for n in mine})
        weight_map.update({n: shard for n in mine})
        shards.append(shard)
    (sharded / "model.safetensors.index.json").write_text(json.dumps({"metadata": {}, "weight_map": weight_map}))
    return sharded, whole, shards


def test_a_checkpoint_in_shards_loads_like_the_same_checkpoint_in_one_file(tmp_path):
    """The reference opens one file (weights.rs:24-32); folders of the larger models of the family
    carry an index and shards."""
    sharded, whole, shards = shard_folder(tmp_path, TINY_B, seed=3, pieces=3)
    spec = load_config(sharded).model_spec()
    a = load_weights(sharded, declare_parameters(spec), torch.float32, "cpu")
    b = load_weights(whole, declare_parameters(spec), torch.float32, "cpu")
    assert a.keys() == b.keys() and len(a) > 30
    for name in a:
        assert torch.equal(a[name], b[name]), name
    from paged_llm_rs_amd.engine.engine import checkpoint_dtype

    assert checkpoint_dtype(sharded) == "float32"


def test_a_missing_shard_is_an_io_error_that_names_it(tmp_path):
    from paged_llm_rs_amd.errors import IoError

    sharded, _, shards = shard_folder(tmp_path, TINY_A, seed=0)
    (sharded / shards[1]).unlink()
    spec = load_config(sharded).model_spec()
    with pytest.raises(IoError, match=shards[1]):
        load_weights(sharded, declare_parameters(spec), torch.float32, "cpu")
    with pytest.raises(IoError, match="model.safetensors"):         # neither one file nor an index
        load_weights(tmp_path, declare_parameters(spec), torch.float32, "cpu")


def test_the_one_report_covers_all_shards(tmp_path):
    sharded, _, shards = shard_folder(tmp_path, TINY_B, seed=1)
    index = json.loads((sharded / "model.safetensors.index.json").read_text())
    # a tensor of the wrong shape in one shard, an unknown one in the other, a missing one in the index
    first = SafetensorsFile(sharded / shards[0])
    tensors = {n: first.tensor(n).clone() for n in first.names()}
    victim = next(n for n in tensors if n.endswith("k_norm.weight"))
    tensors[victim] = torch.zeros(96)
    write_safetensors(sharded / shards[0], tensors)
    second = SafetensorsFile(sharded / shards[1])
    tensors = {n: second.tensor(n).clone() for n in second.names()}
    tensors["model.layers.0.self_attn.rotary_emb.inv_freq"] = torch.zeros(16)
    gone = next(n for n in tensors if n.endswith("down_proj.weight"))
    del tensors[gone]
    write_safetensors(sharded / shards[1], tensors)
    index["weight_map"]["model.layers.0.self_attn.rotary_emb.inv_freq"] = shards[1]
    del index["weight_map"][gone]
    (sharded / "model.safetensors.index.json").write_text(json.dumps(index))
    spec = load_config(sharded).model_spec()
    with pytest.raises(WeightError) as e:
        load_weights(sharded, declare_parameters(spec), torch.float32, "cpu")
    text = str(e.value)
    assert "index.json" in text and f"missing (1): {gone}" in text
    assert "unexpected (1)" in text and "inv_freq" in text
    assert f"wrong shape (1): {victim} has shape [96], expected [32]" in text
    # an index that names a tensor its shard does not hold is refused as such
    index["weight_map"][gone] = shards[1]
    (sharded / "model.safetensors.index.json").write_text(json.dumps(index))
    with pytest.raises(WeightError, match="do not hold"):
        load_weights(sharded, declare_parameters(spec), torch.float32, "cpu")


# ---- tensors a family's checkpoints carry and the model does not use ------------------------------------

def test_tensors_that_a_spec_says_to_ignore_are_not_unexpected(tmp_path):
    import dataclasses

    d = write_random_model(tmp_path / "m", TINY_A, seed=0, dtype="float32")
    f = SafetensorsFile(d / "model.safetensors")
    tensors = {n: f.tensor(n).clone() for n in f.names()}
    tensors["model.layers.0.self_attn.rotary_emb.inv_freq"] = torch.zeros(8)
    tensors["model.layers.1.self_attn.rotary_emb.inv_freq"] = torch.zeros(8)
    tensors["model.stray.weight"] = torch.zeros(3)
    write_safetensors(d / "model.safetensors", tensors)
    spec = load_config(d).model_spec()
    with pytest.raises(WeightError, match=r"unexpected \(3\)"):
        load_weights(d, declare_parameters(spec), torch.float32, "cpu", ignored=spec.ignored_tensors)
    lenient = dataclasses.replace(spec, ignored_tensors=("*.rotary_emb.inv_freq",))
    with pytest.raises(WeightError, match=r"unexpected \(1\): model.stray.weight"):
        load_weights(d, declare_parameters(lenient), torch.float32, "cpu", ignored=lenient.ignored_tensors)
    lenient = dataclasses.replace(spec, ignored_tensors=("*.rotary_emb.inv_freq", "model.stray.*"))
    w = load_weights(d, declare_parameters(lenient), torch.float32, "cpu", ignored=lenient.ignored_tensors)
    assert "model.stray.weight" not in w and not any("inv_freq" in n for n in w)


# ---- the reference's own checkpoint through the loader ----------------------------------------------------

def test_the_references_own_checkpoint_through_config_declaration_and_shape_check():
    """The part of "the engine on the reference's checkpoint" that needs no GPU: its config.json (rotary base
    nested under rope_parameters, keys the engine does not read, a width of 24 with heads of 16:
    tests/fixtures/tiny/config.json:1-37) through the registry, the declaration of every tensor, the one
    check against the file and the model's construction."""
    from conftest import REFERENCE_FIXTURE
    from paged_llm_rs_amd.parts.model import load_model

    if not (REFERENCE_FIXTURE / "model.safetensors").exists():
        pytest.skip("the reference's fixture is not on this machine")
    config, model = load_model(REFERENCE_FIXTURE, "float32", "cpu")
    assert isinstance(config, Qwen3Config) and config.rope_theta == 1e6
    assert (config.hidden_size, config.num_attention_heads, config.num_key_value_heads, config.head_dim) == (24, 4, 2, 16)
    assert not config.tie_word_embeddings and model.lm_head.weight.shape == (128, 24)
    assert len(model.blocks) == 2 and model.embed_tokens.dtype == torch.float32
    f = SafetensorsFile(REFERENCE_FIXTURE / "model.safetensors")
    declared = {d.name for d in declare_parameters(config.model_spec())}
    assert set(f.names()) == declared                      # 2 + 2 * 11 tensors, none optional left out
    attention = model.blocks[1].mixer
    assert torch.equal(attention.q_gain, f.tensor("model.layers.1.self_attn.q_norm.weight"))
    assert torch.equal(attention.qkv_proj.weight[64:96], f.tensor("model.layers.1.self_attn.k_proj.weight"))


# ---- what a spec names beside the layers ------------------------------------------------------------------

def test_transforms_named_by_a_spec_are_declared_and_built(tmp_path):
    import dataclasses

    from paged_llm_rs_amd.parts import register_embed_transform, register_logit_transform
    from paged_llm_rs_amd.parts.model import DecoderModel

    class Shift:
        @staticmethod
        def declare(spec):
            return [ParamDecl("model.shift.weight", (spec.hidden_size,), "matrix")]

        def __init__(self, spec, params, dtype, device):
            self.by = params["model.shift.weight"]

        def __call__(self, x, batch):
            return x + self.by

    class Halve:
        graph_safe = False

        def __init__(self, spec, params, dtype, device):
            self.factor = spec.extra["factor"]

        def __call__(self, logits, batch):
            return logits * self.factor

    register_embed_transform("toy_shift", Shift)
    register_logit_transform("toy_halve", Halve)
    spec = load_config(TINY_A).model_spec()
    assert not any(d.name == "model.shift.weight" for d in declare_parameters(spec))
    plain = DecoderModel(spec, {d.name: torch.zeros(d.shape) for d in declare_parameters(spec)}, torch.float32, "cpu")
    assert plain.embed_transform is None and plain.logit_transform is None and plain.graph_safe
    named = dataclasses.replace(spec, extra={"embed_transform": "toy_shift", "logit_transform": "toy_halve", "factor": 0.5})
    decls = declare_parameters(named)
    assert any(d.name == "model.shift.weight" and d.shape == (64,) for d in decls)
    model = DecoderModel(named, {d.name: torch.ones(d.shape) for d in decls}, torch.float32, "cpu")
    assert isinstance(model.embed_transform, Shift) and model.logit_transform.factor == 0.5
    assert not model.graph_safe                      # a transform that cannot be captured keeps the model's steps eager
    assert model.portion_limits == (16,)             # what the attention mixers report, not a constant of the engine
    with pytest.raises(UnsupportedError, match="toy_nothing"):
        declare_parameters(dataclasses.replace(spec, extra={"logit_transform": "toy_nothing"}))
