"""One registry from an architecture's name to its configuration and model.

The reference selects among registered architectures by probing the checkpoint's
metadata (src/model/architecture.cpp:31-78) and registers exactly one, automatic,
architecture (src/composition/builtin_runtime.cpp:13-58).  Here the name in
``config.json`` (``architectures[0]``, else ``model_type``) selects an entry; an
unknown name is an error that lists the registered ones.
"""
from __future__ import annotations

import json
import os
from dataclasses import dataclass
from typing import Any, Callable, Dict, List, Mapping

from .spec import ModelSpec


@dataclass(frozen=True)
class Architecture:
    """``read_config`` turns the config.json dictionary into the architecture's typed
    configuration; ``build_spec`` turns that into the parts list."""
    name: str
    read_config: Callable[..., Any]
    build_spec: Callable[[Any], ModelSpec]
    aliases: tuple = ()
    # True: ``read_config(cfg, tensor_shapes)`` also takes the checkpoint's tensor names and
    # shapes (or None), to fill what config.json leaves out
    reads_tensor_shapes: bool = False


_ARCHITECTURES: Dict[str, Architecture] = {}


def register_architecture(arch: Architecture, replace: bool = False) -> None:
    for name in (arch.name,) + tuple(arch.aliases):
        if name in _ARCHITECTURES and not replace:
            raise ValueError(f"architecture '{name}' is already registered")
        _ARCHITECTURES[name] = arch


def registered_architectures() -> List[str]:
    return sorted(_ARCHITECTURES)


def architecture_name(cfg: Mapping[str, Any]) -> str:
    archs = cfg.get("architectures")
    if isinstance(archs, (list, tuple)) and archs:
        return str(archs[0])
    if "model_type" in cfg:
        return str(cfg["model_type"])
    raise ValueError("config.json names no architecture: neither 'architectures' nor "
                     "'model_type' is present")


def find_architecture(cfg: Mapping[str, Any]) -> Architecture:
    name = architecture_name(cfg)
    if name not in _ARCHITECTURES:
        raise ValueError(f"no registered architecture is called '{name}'; registered: "
                         f"{registered_architectures()}")
    return _ARCHITECTURES[name]


def read_config_file(model_dir: str) -> Dict[str, Any]:
    """config.json must lie beside the weights (src/checkpoint/catalog.cpp:58-63).  A
    ``generation_config.json`` beside it overrides ``bos_token_id`` and ``eos_token_id``
    (a number, or a list of numbers) and is ignored if it cannot be read
    (src/checkpoint/catalog.cpp:94-121)."""
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
            for key in ("bos_token_id", "eos_token_id"):
                value = gen.get(key)
                number = lambda v: isinstance(v, (int, float)) and not isinstance(v, bool)
                if number(value):
                    cfg[key] = int(value)
                elif isinstance(value, list):
                    ids = [int(v) for v in value if number(v)]
                    if ids:
                        cfg[key] = ids
    return cfg


def spec_from_config(cfg: Mapping[str, Any], tensor_shapes=None):
    """(typed configuration, ModelSpec) of a config.json dictionary.  ``tensor_shapes``:
    name -> shape of the checkpoint's tensors, for architectures that fill from them what
    config.json leaves out."""
    arch = find_architecture(cfg)
    typed = arch.read_config(cfg, tensor_shapes) if arch.reads_tensor_shapes else arch.read_config(cfg)
    spec = arch.build_spec(typed)
    spec.validate()
    return typed, spec


def _register_builtin() -> None:
    from .lfm2 import Lfm2Config
    register_architecture(Architecture(
        name="Lfm2ForCausalLM", aliases=("lfm2",),
        read_config=Lfm2Config.from_dict, build_spec=lambda c: c.to_spec(),
        reads_tensor_shapes=True))


_register_builtin()
