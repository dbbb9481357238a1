from .base import (BlockSpec, ConfigError, JsonReader, LayerCall, ModelSpec, PartSpec,
                   read_config_json)
from .qwen3 import Qwen3Config
from .defosun import DefosunConfig
from .gimipel import GimipelConfig
from .kapanex import KapanexConfig
from .sinepel import SinepelConfig

__all__ = ["BlockSpec", "ConfigError", "JsonReader", "LayerCall", "ModelSpec", "PartSpec",
           "read_config_json", "Qwen3Config", "SinepelConfig", "KapanexConfig", "GimipelConfig", "DefosunConfig"]
