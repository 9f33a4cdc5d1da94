"""Typed model configurations read from config.json."""

from .base import ConfigError, ModelConfig, read_config_json
from .botulorn import BotulornConfig
from .fiterax import FiteraxConfig
from .gilozen import GilozenConfig
from .qwen2 import Qwen2Config

__all__ = ["BotulornConfig", "ConfigError", "FiteraxConfig", "GilozenConfig", "ModelConfig", "Qwen2Config", "read_config_json"]
