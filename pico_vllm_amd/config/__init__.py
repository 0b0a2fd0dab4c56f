from .model_config import ConfigError, Qwen2Config, read_config_json
from .registry import (Architecture, known_architectures, load_model_description,
                       register_architecture, resolve_architecture)
from . import qwen2 as _qwen2  # registers "Qwen2ForCausalLM"
from . import lerazen as _lerazen  # registers "Lerazen"
from . import nasedra as _nasedra  # registers "Nasedra"
from . import dikolix as _dikolix  # registers "Dikolix"
from . import vagelix as _vagelix  # registers "Vagelix"
from .engine_args import EngineArgs

__all__ = ["ConfigError", "Qwen2Config", "read_config_json", "Architecture", "known_architectures",
           "load_model_description", "register_architecture", "resolve_architecture", "EngineArgs"]
