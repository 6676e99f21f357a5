from .base import ConfigError, KeyReader, architecture_name, read_config_json
from .options import EngineOptions
from .qwen2_moe import Qwen2MoeConfig

__all__ = ["ConfigError", "KeyReader", "architecture_name", "read_config_json",
           "EngineOptions", "Qwen2MoeConfig"]
