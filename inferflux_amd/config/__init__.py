from .base import ConfigError, ModelConfig, read_config_json
from .qwen2 import Qwen2Config
from .registry import (config_from_dict, load_config, plan_for, register_architecture,
                       registered_architectures, resolve_architecture)
