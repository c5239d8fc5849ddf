"""From a model folder to a ready step function.

The reference's path: open the checkpoint, select the architecture, resolve it,
compile the program, upload the weights, size the buffers
(src/checkpoint/bootstrap.cpp:13-21; src/backend/cuda/execution_plan.cpp:19-130;
src/backend/cuda/model/weight_setup.cpp).  The model class is chosen by config.json.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Optional

import torch

from ..cache.manager import CacheManager
from ..config.registry import read_config_file, spec_from_config
from ..parts.base import Runtime
from ..weights.loader import Checkpoint, load_tensors
from .model import Model
from .runner import ModelRunner, Workspace

_DTYPES = {"bfloat16": torch.bfloat16, "bf16": torch.bfloat16,
           "float32": torch.float32, "fp32": torch.float32, "f32": torch.float32}


def parse_dtype(name) -> torch.dtype:
    if isinstance(name, torch.dtype):
        if name not in (torch.bfloat16, torch.float32):
            raise ValueError(f"unsupported dtype {name}: bfloat16 or float32")
        return name
    if name not in _DTYPES:
        raise ValueError(f"unknown dtype '{name}': bfloat16 or float32")
    return _DTYPES[name]


@dataclass
class LoadedModel:
    config: object
    spec: object
    model: Model
    cache: CacheManager
    runner: ModelRunner
    rt: Runtime


def make_runtime(device, dtype, ops=None) -> Runtime:
    """The kernels are the HIP ones unless a test passes its own stand-in."""
    if ops is None:
        from ..csrc.hip_ops import HipOps
        ops = HipOps(device)
    return Runtime(device, dtype, ops, Workspace(device))


def read_model_folder(model_dir: str):
    """(typed configuration, ModelSpec) of a model folder: config.json (with
    generation_config.json merged) and, for what it leaves out, the tensors' names and shapes."""
    cfg_dict = read_config_file(model_dir)
    ckpt = Checkpoint(model_dir)
    try:
        return spec_from_config(cfg_dict, {n: tuple(ckpt.info(n).shape) for n in ckpt.names()})
    finally:
        ckpt.close()


def load_model(model_dir: str, *, dtype="bfloat16", device="cuda:0", page_tokens: int = 16,
               n_pages: Optional[int] = None, max_requests: int = 8,
               max_context: Optional[int] = None, max_batched_tokens: int = 2048,
               ops=None, gemm_backend: str = "library") -> LoadedModel:
    """``n_pages``: pages of the cache pool (per group); by default enough for
    ``max_requests`` requests of ``max_context`` tokens.  ``max_context`` defaults to the
    model's own maximum and may not exceed it.  ``gemm_backend``: how bfloat16 steps of more
    than 64 rows multiply: "library" (hipBLASLt, with separate norm and activation kernels)
    or "tiles" (this package's tiled products with the norm, SwiGLU and the residual sum
    folded in, where the sizes allow; the library otherwise)."""
    if gemm_backend not in ("library", "tiles"):
        raise ValueError(f"gemm_backend must be 'library' or 'tiles', not '{gemm_backend}'")
    dtype = parse_dtype(dtype)
    cfg_dict = read_config_file(model_dir)
    ckpt = Checkpoint(model_dir)
    try:
        config, spec = spec_from_config(cfg_dict, {n: tuple(ckpt.info(n).shape) for n in ckpt.names()})
    except Exception:
        ckpt.close()
        raise
    if max_context is None:
        max_context = spec.max_context
    try:
        if max_context > spec.max_context:
            raise ValueError(f"--context {max_context} exceeds model maximum {spec.max_context}")
        model = Model(spec)
        rt = make_runtime(device, dtype, ops)
        rt.use_tiled_products = gemm_backend == "tiles"
        tensors = load_tensors(ckpt, model.expected_tensors(), dtype, device)
    finally:
        ckpt.close()
    model.load(tensors, rt)
    del tensors
    pages_per_request = (max_context + page_tokens - 1) // page_tokens
    if n_pages is None:
        n_pages = pages_per_request * max_requests
    cache = CacheManager(model.cache_layout(), page_tokens=page_tokens, n_pages=n_pages,
                         max_requests=max_requests, max_context=max_context, device=device,
                         dtype=dtype)
    runner = ModelRunner(model, cache, rt, max_batched_tokens=max_batched_tokens)
    return LoadedModel(config, spec, model, cache, runner, rt)
