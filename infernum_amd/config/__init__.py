from .base import ConfigError, UnsupportedModelError, read_config_json
from .llama import Llama3RopeScaling, LlamaConfig
from .registry import (config_from_dict, load_config, model_spec_for, register_architecture, registered_architectures,
                       resolve_architecture)
