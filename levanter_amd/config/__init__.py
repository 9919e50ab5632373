from .lm_config import ConfigError, LmConfig
from .gpt2 import Gpt2Config
from .engine_config import InferenceEngineConfig

__all__ = ["ConfigError", "LmConfig", "Gpt2Config", "InferenceEngineConfig"]
