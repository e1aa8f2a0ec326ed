"""Typed configurations read from a model folder's config.json."""
from .base import ConfigError, ModelConfig, read_config_json
from .llama import LlamaConfig, RopeScaling
from .mifidra import MifidraConfig
from .sofinex import SofinexConfig
from .vafodra import VafodraConfig
from .vupelorn import VupelornConfig

__all__ = ["ConfigError", "ModelConfig", "read_config_json", "LlamaConfig", "MifidraConfig", "RopeScaling", "SofinexConfig", "VafodraConfig", "VupelornConfig"]
