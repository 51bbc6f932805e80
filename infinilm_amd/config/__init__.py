from .errors import ConfigError
from .registry import (load_model_config, read_config_json, register_architecture, registered_architectures,
                       resolve_architecture)
from .spec import HeadSpec, LayerRun, LayerSpec, ModelSpec, PartSpec

__all__ = ["ConfigError", "HeadSpec", "LayerRun", "LayerSpec", "ModelSpec", "PartSpec", "load_model_config",
           "read_config_json", "register_architecture", "registered_architectures", "resolve_architecture"]
