from .spec import PartSpec, LayerSpec, RunStep, ModelSpec
from .lfm2 import Lfm2Config, ConfigError, feed_forward_width
from .registry import (Architecture, register_architecture, registered_architectures,
                       find_architecture, architecture_name, read_config_file,
                       spec_from_config)

__all__ = [
    "PartSpec", "LayerSpec", "RunStep", "ModelSpec", "Lfm2Config", "ConfigError",
    "feed_forward_width", "Architecture", "register_architecture",
    "registered_architectures", "find_architecture", "architecture_name",
    "read_config_file", "spec_from_config",
]
