"""Weights by tensor name: opening a model folder, checking it against what the
model's parts expect, and bringing the tensors to the device.

The reference opens a single ``model.safetensors``, a sharded
``model.safetensors.index.json`` or an explicit file
(src/checkpoint/repositories/safetensors.cpp:24-83), reads tensors by name
(include/celeg/checkpoint/weight_repository.hpp:14-20) and reports binding
problems tensor by tensor (src/model/inference/support.cpp:23-55).  Here ALL
problems of a checkpoint are gathered into one error: missing tensors, tensors
nobody asked for, and wrong shapes.

Dtypes: floating tensors stored in 16-bit are held in bfloat16 by a bfloat16 engine
and widened by a 32-bit engine; a tensor stored in 32-bit stays 32-bit; integer
tensors become int32; "vector" tensors (norm scales, biases, filter taps) are always
widened to 32-bit, which is exact.
"""
from __future__ import annotations

import json
import os
from typing import Dict, List, Mapping

import torch

from ..parts.base import WeightSpec
from .safetensors_io import SafetensorsError, SafetensorsFile, TensorInfo


class WeightError(ValueError):
    """The checkpoint does not fit the model.  ``missing``, ``unexpected`` and
    ``wrong_shape`` hold the details that the message lists."""

    def __init__(self, message, missing=(), unexpected=(), wrong_shape=()):
        super().__init__(message)
        self.missing = list(missing)
        self.unexpected = list(unexpected)
        self.wrong_shape = list(wrong_shape)


class Checkpoint:
    """The tensors of a model folder, across shards."""

    def __init__(self, model_dir: str):
        self.model_dir = model_dir
        single = os.path.join(model_dir, "model.safetensors")
        index = os.path.join(model_dir, "model.safetensors.index.json")
        self._files: Dict[str, SafetensorsFile] = {}
        self._where: Dict[str, str] = {}
        if os.path.isfile(single):
            self._add_file(single)
        elif os.path.isfile(index):
            with open(index) as fh:
                weight_map = json.load(fh).get("weight_map", {})
            for name, shard in weight_map.items():
                path = os.path.join(model_dir, shard)
                if path not in self._files:
                    if not os.path.isfile(path):
                        raise SafetensorsError(f"missing safetensors shard: {path}")
                    self._files[path] = SafetensorsFile(path)
                if name not in self._files[path].tensors:
                    raise SafetensorsError(f"missing tensor: {name} (index names shard {shard})")
                self._where[name] = path
        elif os.path.isfile(model_dir) and model_dir.endswith(".safetensors"):
            self._add_file(model_dir)
        else:
            raise FileNotFoundError("no model.safetensors or model.safetensors.index.json "
                                    f"found in {model_dir}")

    def _add_file(self, path: str) -> None:
        f = SafetensorsFile(path)
        self._files[path] = f
        for name in f.names():
            self._where[name] = path

    def names(self) -> List[str]:
        return list(self._where)

    def info(self, name: str) -> TensorInfo:
        if name not in self._where:
            raise SafetensorsError(f"missing tensor: {name}")
        return self._files[self._where[name]].tensors[name]

    def tensor(self, name: str) -> torch.Tensor:
        if name not in self._where:
            raise SafetensorsError(f"missing tensor: {name}")
        return self._files[self._where[name]].tensor(name)

    def close(self) -> None:
        for f in self._files.values():
            f.close()


def check_tensors(ckpt: Checkpoint, expected: Mapping[str, WeightSpec]) -> None:
    """Raise one ``WeightError`` that lists every missing tensor, every tensor the model
    has no use for and every wrong shape."""
    have = set(ckpt.names())
    missing = sorted(n for n in expected if n not in have)
    unexpected = sorted(n for n in have if n not in expected)
    wrong = []
    for name, spec in expected.items():
        if name in have:
            shape = tuple(ckpt.info(name).shape)
            if shape != tuple(spec.shape) and shape not in [tuple(s) for s in spec.also]:
                wrong.append((name, shape, tuple(spec.shape)))
            elif not ckpt.info(name).is_float:
                wrong.append((name, f"dtype {ckpt.info(name).dtype}", "a floating dtype"))
    if not (missing or unexpected or wrong):
        return
    lines = [f"checkpoint {ckpt.model_dir} does not fit the model:"]
    if missing:
        lines.append(f"  missing tensors ({len(missing)}): " + ", ".join(missing))
    if unexpected:
        lines.append(f"  unexpected tensors ({len(unexpected)}): " + ", ".join(unexpected))
    for name, got, want in wrong:
        lines.append(f"  wrong shape: {name} is {got}, expected {want}")
    raise WeightError("\n".join(lines), missing, unexpected, wrong)


def convert(t: torch.Tensor, kind: str, engine_dtype: torch.dtype) -> torch.Tensor:
    if not t.is_floating_point():
        return t.to(torch.int32)
    if kind == "vector" or engine_dtype == torch.float32 or t.dtype == torch.float32:
        return t.to(torch.float32)
    return t.to(torch.bfloat16)


def load_tensors(ckpt: Checkpoint, expected: Mapping[str, WeightSpec],
                 engine_dtype: torch.dtype, device) -> Dict[str, torch.Tensor]:
    check_tensors(ckpt, expected)
    out = {}
    for name, spec in expected.items():
        out[name] = convert(ckpt.tensor(name), spec.kind, engine_dtype).to(device).contiguous()
    return out
