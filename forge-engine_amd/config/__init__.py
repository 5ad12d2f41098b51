"""Typed configurations: the model's (read from config.json) and the engine's."""

from .engine import EngineConfig, SchedulerConfig
from .model import ConfigError, ModelConfig, load_model_config
from .dubizen import DubizenConfig
from .malusun import MalusunConfig
from .mazanex import MazanexConfig
from .qwen3 import Qwen3Config
from .rekezen import RekezenConfig

__all__ = ["ConfigError", "DubizenConfig", "EngineConfig", "MalusunConfig", "MazanexConfig", "ModelConfig", "Qwen3Config", "RekezenConfig", "SchedulerConfig",
           "load_model_config"]
