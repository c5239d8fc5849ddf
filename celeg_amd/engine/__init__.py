from .batch import StepEntry, StepBatch
from .model import Model
from .runner import ModelRunner, Workspace
from .loading import load_model, LoadedModel, make_runtime, parse_dtype

__all__ = ["StepEntry", "StepBatch", "Model", "ModelRunner", "Workspace", "load_model",
           "LoadedModel", "make_runtime", "parse_dtype"]
