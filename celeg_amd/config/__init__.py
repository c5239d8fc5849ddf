from .spec import PartSpec, LayerSpec, RunStep, ModelSpec
from .registry import (ConfigError, Lfm2Config, feed_forward_width, register_architecture,
                       registered_architectures, read_config_file, read_model_folder, spec_from_config)

__all__ = ["PartSpec", "LayerSpec", "RunStep", "ModelSpec", "Lfm2Config", "ConfigError",
           "feed_forward_width", "register_architecture", "registered_architectures",
           "read_config_file", "read_model_folder", "spec_from_config"]
