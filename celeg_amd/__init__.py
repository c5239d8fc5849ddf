"""celeg_amd: a single-GPU inference engine for MI355X (gfx950), built from parts.

The engine itself is a C++/HIP library (``csrc/``: the kernels, and ``csrc/host``: configuration,
weights, parts, cache manager, step function, scheduler, sampler, C interface); this package is
its Python entry point, a thin layer of ``ctypes`` calls (``native.py``) in the shapes a Python
user expects."""
from .config import (Lfm2Config, ModelSpec, PartSpec, LayerSpec, RunStep, register_architecture,
                     registered_architectures, spec_from_config)

__version__ = "0.2.0"


def __getattr__(name):
    if name in ("Engine", "load_model"):
        from . import engine
        return getattr(engine, name)
    raise AttributeError(f"module 'celeg_amd' has no attribute '{name}'")
