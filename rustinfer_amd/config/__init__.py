from .model_config import ConfigError, LlamaConfig, ModelConfig, RopeScaling, read_config_json
from .registry import (ArchitectureEntry, load_model_config, register_architecture,
                       registered_architectures, resolve_architecture, unregister_architecture)
from .engine_config import EngineConfig, load_engine_config, parse_toml
