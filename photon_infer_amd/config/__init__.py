from .base import ConfigReader, architecture_name, read_config_json
from .dafidra import DafidraConfig
from .dokanex import DokanexConfig
from .llama import LlamaConfig, RopeScaling
from .muretar import MuretarConfig
from .rorevik import RorevikConfig

__all__ = ["ConfigReader", "architecture_name", "read_config_json", "LlamaConfig", "RopeScaling", "DafidraConfig", "RorevikConfig", "DokanexConfig", "MuretarConfig"]
