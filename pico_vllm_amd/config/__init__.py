from .model_config import ConfigError, Qwen2Config, read_config_json
from .registry import (Architecture, known_architectures, load_model_description,
                       register_architecture, resolve_architecture)
from . import qwen2 as _qwen2  # registers "Qwen2ForCausalLM"
from .engine_args import EngineArgs

__all__ = ["ConfigError", "Qwen2Config", "read_config_json", "Architecture", "known_architectures",
           "load_model_description", "register_architecture", "resolve_architecture", "EngineArgs"]
