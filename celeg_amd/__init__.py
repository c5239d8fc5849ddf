"""celeg_amd: a single-GPU inference engine for MI355X (gfx950), built from parts."""
from . import parts  # registers the built-in parts  # noqa: F401
from .config import (Lfm2Config, ModelSpec, PartSpec, LayerSpec, RunStep, register_architecture,
                     registered_architectures, spec_from_config)

__version__ = "0.1.0"


def __getattr__(name):
    # the engine pulls in the GPU side; it is loaded when first asked for
    if name in ("Engine", "load_model"):
        from . import engine
        return getattr(engine, name)
    raise AttributeError(f"module 'celeg_amd' has no attribute '{name}'")
