from .lm_config import ConfigError, LmConfig
from .gpt2 import Gpt2Config
from .zederax import ZederaxConfig
from .nakurax import NakuraxConfig
from .tativik import TativikConfig
from .kegetar import KegetarConfig
from .engine_config import InferenceEngineConfig

__all__ = ["ConfigError", "LmConfig", "Gpt2Config", "ZederaxConfig", "NakuraxConfig", "TativikConfig", "KegetarConfig", "InferenceEngineConfig"]
