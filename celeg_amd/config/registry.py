"""Configuration and the architecture registry, as the library sees them.

Reading config.json (with generation_config.json merged), the typed LFM2 configuration, its
validation and the parts list are the library's (``csrc/host/config.cpp``); here are the Python
views of their results and the way to register an architecture written in Python.
"""
from __future__ import annotations

import json
import os
from dataclasses import dataclass
from typing import Any, Callable, Dict, List, Mapping, Optional, Tuple

from .. import native
from .spec import ModelSpec


class ConfigError(ValueError):
    """A configuration that cannot be built; the message names the key."""


def _describe(cfg: Mapping[str, Any], tensor_shapes=None) -> Dict[str, Any]:
    try:
        return native.describe_config(dict(cfg), tensor_shapes)
    except native.NativeArgumentError as err:
        raise ConfigError(str(err)) from None


# Typed views of configurations, by architecture: a function from the library's typed configuration
# (a dictionary) to whatever Python object stands for it.  An architecture without a view is seen
# as the dictionary itself.  The generic code below and the engine ask this table only.
_typed_views: Dict[str, Callable[[Mapping[str, Any]], Any]] = {}


def register_typed_view(architecture: str, view: Callable[[Mapping[str, Any]], Any]) -> None:
    _typed_views[architecture] = view


def typed_config(architecture: str, config: Mapping[str, Any]):
    view = _typed_views.get(architecture)
    return view(config) if view else config


@dataclass(frozen=True)
class Lfm2Config:
    """The typed LFM2 configuration: every key the library reads, defaults filled in."""
    vocab_size: int
    hidden_size: int
    num_hidden_layers: int
    num_attention_heads: int
    num_key_value_heads: int
    head_dim: int
    intermediate_size: int
    layer_types: Tuple[str, ...]
    conv_L_cache: int
    conv_bias: bool
    rope_theta: float
    norm_eps: float
    max_position_embeddings: int
    block_auto_adjust_ff_dim: bool
    block_multiple_of: int
    block_ffn_dim_multiplier: Optional[float]
    tie_word_embeddings: bool
    bos_token_id: int
    eos_token_ids: Tuple[int, ...]
    pad_token_id: int
    ff_dim: int
    architecture: str = "Lfm2ForCausalLM"

    @classmethod
    def from_typed(cls, c: Mapping[str, Any]) -> "Lfm2Config":
        return cls(c["vocab_size"], c["hidden_size"], c["num_hidden_layers"], c["num_attention_heads"],
                   c["num_key_value_heads"], c["head_dim"], c["intermediate_size"], tuple(c["layer_types"]),
                   c["conv_L_cache"], c["conv_bias"], float(c["rope_theta"]), float(c["norm_eps"]),
                   c["max_position_embeddings"], c["block_auto_adjust_ff_dim"], c["block_multiple_of"],
                   c["block_ffn_dim_multiplier"], c["tie_word_embeddings"], c["bos_token_id"],
                   tuple(c["eos_token_id"]), c["pad_token_id"], c["ff_dim"])

    @classmethod
    def from_dict(cls, cfg: Mapping[str, Any], tensor_shapes=None) -> "Lfm2Config":
        cfg = dict(cfg)
        cfg.setdefault("architectures", [cls.architecture])
        return cls.from_typed(_describe(cfg, tensor_shapes)["config"])

    def to_dict(self) -> Dict[str, Any]:
        out = {k: (list(v) if isinstance(v, tuple) else v) for k, v in vars(self).items()
               if k not in ("ff_dim", "architecture", "eos_token_ids")}
        out["architectures"] = [self.architecture]
        out["model_type"] = "lfm2"
        out["eos_token_id"] = list(self.eos_token_ids) if len(self.eos_token_ids) != 1 else self.eos_token_ids[0]
        return out


register_typed_view(Lfm2Config.architecture, Lfm2Config.from_typed)


def feed_forward_width(intermediate_size: int, auto_adjust: bool, multiple_of: int,
                       multiplier: Optional[float]) -> int:
    """The SwiGLU width the library computes for these keys."""
    cfg = {"architectures": [Lfm2Config.architecture], "vocab_size": 8, "hidden_size": 8, "num_hidden_layers": 1,
           "num_attention_heads": 1, "layer_types": ["conv"], "conv_L_cache": 1, "rope_theta": 1.0,
           "max_position_embeddings": 8, "intermediate_size": intermediate_size,
           "block_auto_adjust_ff_dim": auto_adjust, "block_multiple_of": multiple_of,
           "block_ffn_dim_multiplier": multiplier}
    return _describe(cfg)["config"]["ff_dim"]


def registered_architectures() -> List[str]:
    return native.registered("architectures")


def register_architecture(name: str, build: Callable[[Dict[str, Any], Optional[Dict[str, Any]]], Any]) -> None:
    """``build(config: dict, tensor_shapes: dict or None)`` returns a ``ModelSpec`` (or a pair
    (typed configuration dict, ModelSpec))."""
    def describe(config, shapes):
        result = build(config, shapes)
        typed, spec = result if isinstance(result, tuple) else (dict(config), result)
        return {"config": typed, "spec": spec.to_json()}
    native.register_architecture(name, describe)


def read_config_file(model_dir: str) -> Dict[str, Any]:
    """config.json of a model folder as a dictionary, generation_config.json merged the way the
    library merges it (src/checkpoint/catalog.cpp:94-121): what tools print."""
    path = os.path.join(model_dir, "config.json")
    if not os.path.isfile(path):
        raise FileNotFoundError(f"config.json not found in model folder {model_dir}")
    with open(path) as fh:
        cfg = json.load(fh)
    generation = os.path.join(model_dir, "generation_config.json")
    if os.path.isfile(generation):
        try:
            with open(generation) as fh:
                gen = json.load(fh)
        except (OSError, ValueError):
            gen = None
        if isinstance(gen, dict):
            number = lambda v: isinstance(v, (int, float)) and not isinstance(v, bool)
            for key in ("bos_token_id", "eos_token_id"):
                value = gen.get(key)
                if number(value):
                    cfg[key] = int(value)
                elif isinstance(value, list):
                    ids = [int(v) for v in value if number(v)]
                    if ids:
                        cfg[key] = ids
    return cfg


def _typed(described: Dict[str, Any]):
    return typed_config(described["spec"]["architecture"], described["config"])


def spec_from_config(cfg: Mapping[str, Any], tensor_shapes=None):
    """(typed configuration, ModelSpec) of a config.json dictionary."""
    d = _describe(cfg, tensor_shapes)
    return _typed(d), ModelSpec.from_json(d["spec"])


def read_model_folder(model_dir: str):
    """(typed configuration, ModelSpec, expected tensors) of a model folder."""
    try:
        d = native.describe_folder(model_dir)
    except native.NativeArgumentError as err:
        if "not found" in str(err):
            raise FileNotFoundError(str(err)) from None
        raise ConfigError(str(err)) from None
    return _typed(d), ModelSpec.from_json(d["spec"]), d["expected_tensors"]
