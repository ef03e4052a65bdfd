from .engine_config import EngineConfig
from .model_config import ConfigError, LlamaConfig, ModelConfig, read_config_json
from .zifelorn_config import ZifelornConfig
from .vezodra_config import VezodraConfig
from .mutusun_config import MutusunConfig
from .labirax_config import LabiraxConfig
from .registry import (Architecture, architecture_for, architecture_of, known_architectures, known_shapes,
                       load_model_config, shape_config, register_architecture, unregister_architecture)

__all__ = ["EngineConfig", "ConfigError", "LlamaConfig", "ModelConfig", "ZifelornConfig", "VezodraConfig", "MutusunConfig", "LabiraxConfig",
           "read_config_json", "Architecture",
           "architecture_for", "architecture_of", "known_architectures", "known_shapes", "shape_config", "load_model_config",
           "register_architecture", "unregister_architecture"]
