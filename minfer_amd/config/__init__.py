from .base import ConfigError, KeyReader, architecture_name, read_config_json
from .qwen2 import Qwen2Config

__all__ = ["ConfigError", "KeyReader", "Qwen2Config", "architecture_name", "read_config_json"]
