from .base import ConfigReader, architecture_name, read_config_json
from .llama import LlamaConfig, RopeScaling

__all__ = ["ConfigReader", "architecture_name", "read_config_json", "LlamaConfig", "RopeScaling"]
