from .base import ConfigError, ModelConfig, read_config_json
from .mumusun import MumusunConfig
from .podurax import PoduraxConfig
from .qwen2 import Qwen2Config
from .tabatar import TabatarConfig
from .vavadra import VavadraConfig
from .registry import (config_from_dict, load_config, plan_for, register_architecture,
                       registered_architectures, resolve_architecture)
