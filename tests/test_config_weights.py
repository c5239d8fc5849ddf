"""Configuration, registry, safetensors reading and writing, weight errors, random weights."""
import json
import os
import struct

import pytest
import torch

import plain_lfm2 as plain
from conftest import TINY, TINY_A, TINY_B
from helpers import reordered_lfm2

from celeg_amd import native
from celeg_amd.config import (ConfigError, Lfm2Config, ModelSpec, PartSpec, RunStep, register_architecture,
                              registered_architectures, spec_from_config)
from celeg_amd.weights import (SafetensorsError, SafetensorsFile, WeightError, check_folder, write_random_model,
                               write_safetensors)


# ---------------------------------------------------------------- configuration
def test_config_reads_every_key():
    a, b = Lfm2Config.from_dict(TINY_A), Lfm2Config.from_dict(TINY_B)
    assert (a.hidden_size, a.num_attention_heads, a.num_key_value_heads, a.head_dim) == (64, 4, 2, 16)
    assert a.ff_dim == 192 and b.ff_dim == 352
    assert a.conv_L_cache == 3 and b.conv_L_cache == 4 and b.conv_bias and not a.conv_bias
    assert a.tie_word_embeddings and not b.tie_word_embeddings
    assert a.norm_eps == 1e-5 and b.norm_eps == 1e-6
    assert a.eos_token_ids == (7,) and b.eos_token_ids == (2, 3)
    assert b.rope_theta == 1e6 and a.max_position_embeddings == 128


def test_ff_arithmetic_of_the_published_shapes():
    def ff(inter, mult):
        cfg = dict(TINY_B, intermediate_size=inter, block_multiple_of=mult)
        return Lfm2Config.from_dict(cfg).ff_dim
    assert ff(6656, 256) == 4608 and ff(12288, 256) == 8192 and ff(10752, 256) == 7168
    assert ff(512, 32) == 352
    for inter, mult in [(6656, 256), (512, 32), (1000, 7)]:
        assert ff(inter, mult) == plain.ff_dim(inter, True, mult, 1.0)


def test_config_defaults_and_aliases():
    cfg = {k: v for k, v in TINY_A.items() if k not in ("num_key_value_heads", "head_dim", "norm_eps")}
    c = Lfm2Config.from_dict(dict(cfg, rms_norm_eps=2e-5))
    assert c.num_key_value_heads == 4 and c.head_dim == 16 and c.norm_eps == 2e-5
    assert Lfm2Config.from_dict(cfg).norm_eps == 1e-6
    with pytest.raises(ConfigError, match="disagree"):
        Lfm2Config.from_dict(dict(TINY_A, rms_norm_eps=1e-3))


def _shapes(cfg):
    return {e["name"]: tuple(e["shape"]) for e in _expected(cfg)}


def test_keys_the_reference_accepts_in_other_places(tmp_path):
    """rope_theta under rope_parameters (src/model/inference/metadata.cpp:427-429), the
    original LFM2 keys full_attn_idxs and block_ff_dim, layer kinds and the feed-forward
    width from the checkpoint's tensors when config.json is silent
    (src/model/inference/rules.cpp:18-26, rules_attention.cpp:138-160,
    global_facts.cpp:127-152), and generation_config.json overriding the end tokens
    (src/checkpoint/catalog.cpp:94-121)."""
    from celeg_amd.config import read_config_file
    from celeg_amd.config import read_model_folder
    base = Lfm2Config.from_dict(TINY_B)
    # a config.json as newer writers lay it out: no top-level rope_theta
    nested = {k: v for k, v in TINY_B.items() if k != "rope_theta"}
    nested["rope_parameters"] = {"rope_theta": 1000000.0, "rope_type": "default"}
    assert Lfm2Config.from_dict(nested) == base
    with pytest.raises(ConfigError, match="disagree"):
        Lfm2Config.from_dict(dict(nested, rope_theta=5.0))
    # the original keys
    old = {k: v for k, v in TINY_B.items() if k not in ("layer_types", "intermediate_size")}
    old.update(full_attn_idxs=[2, 4], block_ff_dim=512)
    assert Lfm2Config.from_dict(old) == base
    with pytest.raises(ConfigError, match="full_attn_idxs"):
        Lfm2Config.from_dict(dict(old, full_attn_idxs=[2, 6]))
    with pytest.raises(ConfigError, match="disagree"):
        Lfm2Config.from_dict(dict(old, intermediate_size=500))
    # silent config: kinds and width from the tensors
    silent = {k: v for k, v in TINY_B.items() if k not in ("layer_types", "intermediate_size")}
    got = Lfm2Config.from_dict(silent, _shapes(TINY_B))
    assert got.layer_types == base.layer_types and got.ff_dim == base.ff_dim == 352
    with pytest.raises(ConfigError, match="layer_types"):
        Lfm2Config.from_dict(silent)                       # nothing to infer from
    with pytest.raises(ConfigError, match="intermediate_size"):
        Lfm2Config.from_dict(dict(silent, layer_types=list(base.layer_types)))
    shapes = _shapes(TINY_B)
    del shapes["model.layers.3.conv.in_proj.weight"]
    with pytest.raises(ConfigError, match=r"layer\(s\) \[3\]"):
        Lfm2Config.from_dict(silent, shapes)
    # a layer_types that contradicts the tensors
    wrong = list(base.layer_types)
    wrong[0], wrong[2] = wrong[2], wrong[0]
    with pytest.raises(ConfigError, match=r"'layer_types'\[0\]"):
        Lfm2Config.from_dict(dict(TINY_B, layer_types=wrong), _shapes(TINY_B))
    # through a folder: the silent config loads, and generation_config.json wins
    folder = write_random_model(TINY_B, str(tmp_path / "m"), seed=0, dtype=torch.float32)
    json.dump(silent, open(os.path.join(folder, "config.json"), "w"))
    json.dump({"bos_token_id": 9, "eos_token_id": [11, 12, "x"], "temperature": 0.3},
              open(os.path.join(folder, "generation_config.json"), "w"))
    config, spec, _ = read_model_folder(folder)
    assert config.layer_types == base.layer_types and config.ff_dim == 352
    assert config.eos_token_ids == (11, 12) and config.bos_token_id == 9 and spec.eos_token_ids == (11, 12)
    json.dump({"eos_token_id": 5}, open(os.path.join(folder, "generation_config.json"), "w"))
    assert read_config_file(folder)["eos_token_id"] == 5 and read_config_file(folder)["bos_token_id"] == 0
    open(os.path.join(folder, "generation_config.json"), "w").write("{ not json")
    assert read_config_file(folder)["eos_token_id"] == [2, 3]     # unreadable: ignored


@pytest.mark.parametrize("key", ["vocab_size", "hidden_size", "num_hidden_layers",
                                 "num_attention_heads", "rope_theta", "conv_L_cache",
                                 "layer_types", "intermediate_size", "max_position_embeddings"])
def test_missing_key_is_named(key):
    cfg = {k: v for k, v in TINY_A.items() if k != key}
    with pytest.raises(ConfigError, match=key):
        Lfm2Config.from_dict(cfg)


@pytest.mark.parametrize("change,word", [
    ({"num_key_value_heads": 3}, "multiple"), ({"head_dim": 15}, "even"),
    ({"layer_types": ["conv"]}, "layer_types"), ({"layer_types": ["conv", "mamba", "conv", "conv"]}, "mamba"),
    ({"conv_L_cache": 0}, "conv_L_cache"), ({"hidden_size": "64"}, "integer"),
    ({"num_key_value_heads": 4, "head_dim": 32}, "exceeds"), ({"norm_eps": 0.0}, "norm_eps")])
def test_invalid_config_is_refused(change, word):
    with pytest.raises(ConfigError, match=word):
        Lfm2Config.from_dict(dict(TINY_A, **change))


def test_registry_chooses_by_name_and_lists_names_on_a_miss():
    assert "Lfm2ForCausalLM" in registered_architectures()
    config, spec = spec_from_config(TINY_B)
    assert isinstance(config, Lfm2Config) and isinstance(spec, ModelSpec)
    assert [l.mixer.kind for l in spec.layers] == ["short_conv", "short_conv", "gqa_attention",
                                                   "short_conv", "gqa_attention", "short_conv"]
    assert spec.head.kind == "linear_head" and spec_from_config(TINY_A)[1].head.kind == "tied_head"
    with pytest.raises(ValueError, match="Lfm2ForCausalLM"):
        spec_from_config(dict(TINY_A, architectures=["NopeForCausalLM"]))
    only_type = {k: v for k, v in TINY_A.items() if k != "architectures"}
    assert spec_from_config(only_type)[1].architecture == "Lfm2ForCausalLM"


def test_spec_sizes_come_from_the_config_only():
    _, spec = spec_from_config(TINY_B)
    att = spec.layers[2].mixer.params
    assert (att["heads"], att["kv_heads"], att["head_dim"], att["eps"]) == (4, 1, 32, 1e-6)
    assert att["position"].params["theta"] == 1e6
    assert spec.layers[0].mixer.params == {"width": 128, "taps": 4, "bias": True}
    assert spec.layers[0].ffn.params == {"width": 128, "ff": 352}
    assert spec.layers[0].mixer.tensors["conv_bias"] == "model.layers.0.conv.conv.bias"


def test_run_order_validation():
    reordered_lfm2()
    def describe(order):
        return native.describe_config(dict(TINY_A, architectures=["Lfm2Reordered"], run_order=order))
    with pytest.raises(native.NativeArgumentError, match="does not run before"):
        describe([[0, None], [1, 1]])
    with pytest.raises(native.NativeArgumentError, match="names layer 9"):
        describe([[9, None]])
    with pytest.raises(native.NativeArgumentError, match="keys and values"):
        describe([[0, None], [1, None], [2, 1]])             # a convolution cannot read a cache
    # a layer named twice and one that reads another's cache
    d = describe([[0, None], [1, None], [1, None], [3, 1]])
    layout = d["cache_layout"]
    assert [g["layers"] for g in layout["kv_groups"]] == [2]
    assert [(u["step"], u["group"], u["layer"], u["writes"]) for u in layout["kv_of_step"]] == \
        [(1, 0, 0, True), (2, 0, 1, True), (3, 0, 0, False)]
    assert [st["step"] for st in layout["states"]] == [0]
    assert "model.layers.3.self_attn.k_proj.weight" not in [e["name"] for e in d["expected_tensors"]]


# ---------------------------------------------------------------- safetensors
def test_safetensors_round_trip_and_agreement_with_the_library(tmp_path):
    from safetensors import safe_open
    tensors = {"a": torch.randn(3, 5), "b": torch.randn(7).bfloat16(),
               "c": torch.arange(6, dtype=torch.int64).reshape(2, 3), "d": torch.randn(2, 2).half()}
    path = str(tmp_path / "x.safetensors")
    write_safetensors(path, tensors, metadata={"format": "pt"})
    f = SafetensorsFile(path)
    assert sorted(f.names()) == ["a", "b", "c", "d"]
    for name, t in tensors.items():
        assert torch.equal(f.tensor(name), t)
    with safe_open(path, framework="pt") as lib:       # the library reads what we wrote
        for name, t in tensors.items():
            assert torch.equal(lib.get_tensor(name), t)
    with pytest.raises(SafetensorsError, match="missing tensor: zz"):
        f.tensor("zz")
    f.close()


def _raw(path, header: dict, data: bytes):
    text = json.dumps(header).encode()
    with open(path, "wb") as fh:
        fh.write(struct.pack("<Q", len(text)) + text + data)


def _native_reader(path):
    """The library's reader on the same file: a model folder around it."""
    folder = os.path.dirname(path)
    json.dump(TINY_A, open(os.path.join(folder, "config.json"), "w"))
    check_folder(folder)


@pytest.mark.parametrize("SafetensorsFile", [SafetensorsFile, _native_reader], ids=["python", "library"])
def test_malformed_safetensors_files(tmp_path, SafetensorsFile):
    p = str(tmp_path / "model.safetensors")
    with open(p, "wb") as fh:
        fh.write(b"abc")
    with pytest.raises(SafetensorsError, match="too small"):
        SafetensorsFile(p)
    with open(p, "wb") as fh:
        fh.write(struct.pack("<Q", 1 << 40) + b"{}")
    with pytest.raises(SafetensorsError, match="header length"):
        SafetensorsFile(p)
    _raw(p, {"a": {"dtype": "F8_E4M3", "shape": [1], "data_offsets": [0, 1]}}, b"\0")
    with pytest.raises(SafetensorsError, match="unsupported dtype"):
        SafetensorsFile(p)
    _raw(p, {"a": {"dtype": "F32", "shape": [2], "data_offsets": [0, 16]}}, b"\0" * 8)
    with pytest.raises(SafetensorsError, match="out-of-range"):
        SafetensorsFile(p)
    _raw(p, {"a": {"dtype": "F32", "shape": [3], "data_offsets": [0, 8]}}, b"\0" * 8)
    with pytest.raises(SafetensorsError, match="byte count"):
        SafetensorsFile(p)
    _raw(p, {"a": {"dtype": "F32", "shape": [2], "data_offsets": [0, 8]},
             "b": {"dtype": "F32", "shape": [2], "data_offsets": [4, 12]}}, b"\0" * 12)
    with pytest.raises(SafetensorsError, match="overlapping"):
        SafetensorsFile(p)
    text = b'{"a":{"dtype":"F32","shape":[1],"data_offsets":[0,4]},"a":{"dtype":"F32","shape":[1],"data_offsets":[4,8]}}'
    with open(p, "wb") as fh:
        fh.write(struct.pack("<Q", len(text)) + text + b"\0" * 8)
    with pytest.raises(SafetensorsError, match="duplicate"):
        SafetensorsFile(p)


# ---------------------------------------------------------------- weights against a model
def _expected(cfg):
    return native.describe_config(cfg)["expected_tensors"]


def test_one_error_lists_missing_unexpected_and_wrong_shapes(tmp_path):
    folder = write_random_model(TINY_B, str(tmp_path / "m"), seed=3, dtype=torch.float32)
    f = SafetensorsFile(os.path.join(folder, "model.safetensors"))
    tensors = {n: f.tensor(n).clone() for n in f.names()}
    f.close()
    del tensors["model.layers.2.self_attn.q_layernorm.weight"]
    del tensors["lm_head.weight"]
    tensors["model.layers.0.conv.in_proj.weight"] = torch.zeros(5, 5)
    tensors["model.layers.9.extra.weight"] = torch.zeros(1)
    write_safetensors(os.path.join(folder, "model.safetensors"), tensors)
    with pytest.raises(WeightError) as info:
        check_folder(folder)
    err = info.value
    assert err.missing == ["lm_head.weight", "model.layers.2.self_attn.q_layernorm.weight"]
    assert err.unexpected == ["model.layers.9.extra.weight"]
    assert err.wrong_shape == ["model.layers.0.conv.in_proj.weight is (5, 5), expected (384, 128)"]
    text = str(err)
    for word in ("missing tensors (2)", "unexpected tensors (1)", "wrong shape",
                 "model.layers.9.extra.weight", "(5, 5)", "(384, 128)"):
        assert word in text


def test_tensors_nobody_asks_for_are_a_warning_unless_strict(tmp_path):
    """The reference binds tensors by name and leaves the rest alone
    (include/celeg/checkpoint/weight_repository.hpp:14-20; src/checkpoint/formats/safetensors.cpp:283-297
    fails on a missing tensor only): a tied model whose checkpoint still carries lm_head.weight, or an
    exported buffer, is no error.  The description names what is left over; a strict check refuses it."""
    folder = write_random_model(TINY_A, str(tmp_path / "m"), seed=3, dtype=torch.float32)
    path = os.path.join(folder, "model.safetensors")
    f = SafetensorsFile(path)
    tensors = {n: f.tensor(n).clone() for n in f.names()}
    f.close()
    assert "lm_head.weight" not in tensors                     # Tiny A ties its head to the embedding
    tensors["lm_head.weight"] = tensors["model.embed_tokens.weight"].clone()
    tensors["model.rotary_emb.inv_freq"] = torch.zeros(8)
    write_safetensors(path, tensors)
    check_folder(folder)
    assert native.describe_folder(folder)["unused_tensors"] == ["lm_head.weight", "model.rotary_emb.inv_freq"]
    with pytest.raises(WeightError) as info:
        check_folder(folder, strict=True)
    assert info.value.unexpected == ["lm_head.weight", "model.rotary_emb.inv_freq"] and not info.value.missing
    # beside a real fault they are still listed, in the one error
    del tensors["model.layers.0.operator_norm.weight"]
    write_safetensors(path, tensors)
    with pytest.raises(WeightError) as info:
        check_folder(folder)
    assert info.value.missing == ["model.layers.0.operator_norm.weight"]
    assert info.value.unexpected == ["lm_head.weight", "model.rotary_emb.inv_freq"]


def test_conv_filter_is_accepted_in_both_shapes_and_bias_is_required(tmp_path):
    folder = write_random_model(TINY_B, str(tmp_path / "m"), seed=3, dtype=torch.float32)
    path = os.path.join(folder, "model.safetensors")
    f = SafetensorsFile(path)
    tensors = {n: f.tensor(n).clone() for n in f.names()}
    f.close()
    tensors["model.layers.0.conv.conv.weight"] = tensors["model.layers.0.conv.conv.weight"].reshape(128, 4)
    write_safetensors(path, tensors)
    check_folder(folder)
    del tensors["model.layers.1.conv.conv.bias"]
    write_safetensors(path, tensors)
    with pytest.raises(WeightError, match="model.layers.1.conv.conv.bias"):
        check_folder(folder)


def test_dtype_policy(tmp_path):
    folder = write_random_model(TINY_A, str(tmp_path / "m"), seed=0, dtype=torch.bfloat16)
    path = os.path.join(folder, "model.safetensors")
    f = SafetensorsFile(path)
    tensors = {n: f.tensor(n).clone() for n in f.names()}
    f.close()
    kept32 = "model.layers.1.self_attn.out_proj.weight"
    tensors[kept32] = tensors[kept32].float()
    write_safetensors(path, tensors)
    held = native.describe_folder(folder)["held_as"]
    assert held["model.embed_tokens.weight"] == {"stored": "BF16", "bfloat16": "bfloat16", "float32": "float32"}
    assert held[kept32]["bfloat16"] == "float32"                                 # stored in 32-bit: stays so
    assert held["model.layers.0.operator_norm.weight"]["bfloat16"] == "float32"   # vectors widen exactly
    assert held["model.layers.0.conv.conv.weight"]["bfloat16"] == "float32"
    assert all(h["float32"] == "float32" for h in held.values())


def test_random_weights_are_keyed_by_seed_and_name(tmp_path):
    a = write_random_model(TINY_A, str(tmp_path / "a"), seed=0, dtype=torch.float32)
    b = write_random_model(TINY_A, str(tmp_path / "b"), seed=0, dtype=torch.float32)
    c = write_random_model(TINY_A, str(tmp_path / "c"), seed=1, dtype=torch.float32)
    fa, fb, fc = (SafetensorsFile(os.path.join(d, "model.safetensors")) for d in (a, b, c))
    name = "model.layers.1.self_attn.q_proj.weight"
    assert torch.equal(fa.tensor(name), fb.tensor(name))
    assert not torch.equal(fa.tensor(name), fc.tensor(name))
    assert abs(float(fa.tensor(name).std()) - 0.02) < 0.002
    assert abs(float(fa.tensor("model.layers.0.ffn_norm.weight").mean()) - 1.0) < 0.02
    assert sorted(fa.names()) == sorted(e["name"] for e in _expected(TINY_A))
    assert json.load(open(os.path.join(a, "config.json")))["hidden_size"] == 64
    # a folder without weights, a folder without config
    os.remove(os.path.join(a, "model.safetensors"))
    with pytest.raises(FileNotFoundError, match="model.safetensors"):
        check_folder(a)
    from celeg_amd.config import read_config_file
    os.remove(os.path.join(b, "config.json"))
    with pytest.raises(FileNotFoundError, match="config.json"):
        read_config_file(b)


def test_sharded_checkpoint(tmp_path):
    folder = write_random_model(TINY_A, str(tmp_path / "m"), seed=0, dtype=torch.float32)
    path = os.path.join(folder, "model.safetensors")
    f = SafetensorsFile(path)
    names = f.names()
    half = len(names) // 2
    write_safetensors(os.path.join(folder, "s1.safetensors"), {n: f.tensor(n).clone() for n in names[:half]})
    write_safetensors(os.path.join(folder, "s2.safetensors"), {n: f.tensor(n).clone() for n in names[half:]})
    whole = {n: f.tensor(n).clone() for n in names}
    f.close()
    os.remove(path)
    index = {"weight_map": {n: ("s1.safetensors" if i < half else "s2.safetensors")
                            for i, n in enumerate(names)}}
    json.dump(index, open(os.path.join(folder, "model.safetensors.index.json"), "w"))
    check_folder(folder)
    assert set(native.describe_folder(folder)["held_as"]) == set(whole)
    os.remove(os.path.join(folder, "s2.safetensors"))
    with pytest.raises(SafetensorsError, match="missing safetensors shard"):
        check_folder(folder)
