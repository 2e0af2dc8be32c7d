from .base import ConfigError, ModelConfig, key, read_config_json, architecture_name   # noqa: F401
from .gemma2 import Gemma2Config   # noqa: F401
