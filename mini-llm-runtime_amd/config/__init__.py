from .registry import (ConfigError, config_class, config_from_dict, known_architectures,
                       load_config, register_architecture)
from .specs import (AttentionSpec, LayerRun, LayerSpec, MlpSpec, ModelSpec, NormSpec,
                    PositionSpec)
from .qwen3 import Qwen3Config

__all__ = ["ConfigError", "config_class", "config_from_dict", "known_architectures", "load_config",
           "register_architecture", "AttentionSpec", "LayerRun", "LayerSpec", "MlpSpec",
           "ModelSpec", "NormSpec", "PositionSpec", "Qwen3Config"]
