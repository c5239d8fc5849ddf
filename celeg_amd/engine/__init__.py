from .batch import TOKEN_FROM_DEVICE, StepEntry, StepBatch
from .model import Model
from .runner import ModelRunner, Workspace
from .loading import load_model, LoadedModel, make_runtime, parse_dtype, read_model_folder
from .scheduler import (Scheduler, SchedulerOptions, RequestOptions, RequestStatus, Request,
                        PlannedEntry)
from .engine import Engine

__all__ = ["TOKEN_FROM_DEVICE", "StepEntry", "StepBatch", "Model", "ModelRunner", "Workspace", "load_model",
           "LoadedModel", "make_runtime", "read_model_folder", "parse_dtype", "Scheduler", "SchedulerOptions",
           "RequestOptions", "RequestStatus", "Request", "PlannedEntry", "Engine"]
