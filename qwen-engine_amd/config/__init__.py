from .spec import (AttentionSpec, LayerSpec, ModelSpec, RMSNormSpec, RopeSpec,
                   ScheduleEntry, SwiGLUSpec)
from .qwen3 import ConfigError, Qwen3Config
from .registry import (config_from_dict, config_from_folder, known_architectures,
                       register_architecture, unregister_architecture)
from .engine_config import EngineConfig
