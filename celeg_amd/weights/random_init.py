"""The random-weights mode: a model folder (config.json, model.safetensors) written
from a configuration and a seed.

The reference has no such mode (its tests use shapes only,
tests/automatic_inference_test.cpp:13-38).  Every tensor is drawn from a generator
keyed by (seed, tensor name), so a tensor's values do not depend on which other
tensors exist or on the order of writing: matrices, tables, biases and filter taps
are N(0, std); norm scales are 1 + N(0, std).  Values are drawn in 32-bit and then
rounded to the storage dtype.
"""
from __future__ import annotations

import hashlib
import json
import os
from typing import Any, Dict, Mapping

import torch

from .. import native
from .safetensors_io import write_safetensors


def tensor_generator(seed: int, name: str) -> torch.Generator:
    digest = hashlib.sha256(f"{seed}:{name}".encode("utf-8")).digest()
    gen = torch.Generator(device="cpu")
    gen.manual_seed(int.from_bytes(digest[:8], "little") & ((1 << 63) - 1))
    return gen


def random_tensor(seed: int, name: str, shape, init: str, std: float) -> torch.Tensor:
    t = torch.randn(tuple(shape), generator=tensor_generator(seed, name), dtype=torch.float32) * std
    if init == "around_one":
        t = t + 1.0
    elif init != "normal":
        raise ValueError(f"unknown initialisation '{init}'")
    return t


def random_tensors(expected, seed: int, std: float = 0.02,
                   dtype: torch.dtype = torch.bfloat16) -> Dict[str, torch.Tensor]:
    """``expected``: the library's list of the tensors a model wants
    ([{"name", "shape", "init", ..}], ``native.describe_config(..)["expected_tensors"]``)."""
    return {e["name"]: random_tensor(seed, e["name"], e["shape"], e["init"], std).to(dtype) for e in expected}


def write_random_model(config: Mapping[str, Any], out_dir: str, seed: int,
                       dtype: torch.dtype = torch.bfloat16, std: float = 0.02) -> str:
    """Write ``out_dir/config.json`` and ``out_dir/model.safetensors`` for the architecture
    that ``config`` names.  Returns ``out_dir``."""
    from ..config.registry import ConfigError
    try:
        expected = native.describe_config(dict(config))["expected_tensors"]   # the parts know which tensors they want
    except native.NativeArgumentError as err:
        raise ConfigError(str(err)) from None
    os.makedirs(out_dir, exist_ok=True)
    with open(os.path.join(out_dir, "config.json"), "w") as fh:
        json.dump(dict(config), fh, indent=1)
    write_safetensors(os.path.join(out_dir, "model.safetensors"),
                      random_tensors(expected, seed, std, dtype),
                      metadata={"format": "pt", "seed": str(seed)})
    return out_dir
