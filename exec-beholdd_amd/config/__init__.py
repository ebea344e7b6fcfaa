"""Typed configurations read from config.json."""

from .base import ConfigError, ConfigReader, LayerKinds, architecture_name, read_config_json
from .qwen3 import Qwen3Config
from .gokazen import GokazenConfig
from .pudorax import PudoraxConfig
from .dupidra import DupidraConfig
from .vepelix import VepelixConfig

__all__ = ["ConfigError", "ConfigReader", "architecture_name", "read_config_json", "LayerKinds", "Qwen3Config", "GokazenConfig", "PudoraxConfig",
           "DupidraConfig", "VepelixConfig"]
