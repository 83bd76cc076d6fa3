from .errors import ConfigError, WeightError, UnsupportedSizeError
from .spec import PartSpec, BlockSpec, ScheduleEntry, StreamOffset, ModelSpec
from .registry import (register_architecture, unregister_architecture, get_architecture,
                       registered_architectures, architecture_of, read_config, Architecture)
from .qwen2 import Qwen2Config
from .vivevik import VivevikConfig
from .ruvalorn import RuvalornConfig
from .minodra import MinodraConfig
from .ninisun import NinisunConfig

__all__ = [
    "ConfigError", "WeightError", "UnsupportedSizeError", "PartSpec", "BlockSpec",
    "ScheduleEntry", "StreamOffset", "ModelSpec", "register_architecture", "unregister_architecture",
    "get_architecture", "registered_architectures", "architecture_of", "read_config",
    "Architecture", "Qwen2Config", "VivevikConfig", "RuvalornConfig", "MinodraConfig", "NinisunConfig",
]
