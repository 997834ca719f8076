from .engine_config import EngineConfig
from .model_config import ConfigError, ModelConfig, Qwen3Config
from .registry import (Architecture, architecture_of, get_architecture, load_model_config,
                       register_architecture, registered_architectures, unregister_architecture)
