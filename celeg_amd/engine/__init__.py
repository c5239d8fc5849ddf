from .engine import (Engine, LoadedModel, RequestOptions, RequestStatus, Scheduler, SchedulerOptions,
                     StepEntry, load_model, parse_dtype, read_model_folder)

__all__ = ["Engine", "LoadedModel", "RequestOptions", "RequestStatus", "Scheduler", "SchedulerOptions",
           "StepEntry", "load_model", "parse_dtype", "read_model_folder"]
