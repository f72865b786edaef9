from .base import ConfigError, UnsupportedArchitecture, architecture_name, read_config_json
from .qwen3 import Qwen3Config
