from .engine_config import EngineConfig, canonical_dtype
from .registry import (
    DEFAULT_MODEL_DIR,
    Architecture,
    ConfigError,
    architecture_name,
    architectures,
    get_architecture,
    load_model_config,
    read_config_json,
    register_architecture,
)
from .specs import (
    AttentionSpec,
    BlockSpec,
    ModelSpec,
    RMSNormSpec,
    RotarySpec,
    ScheduleEntry,
    SwiGLUSpec,
)

__all__ = [
    "DEFAULT_MODEL_DIR",
    "Architecture",
    "AttentionSpec",
    "BlockSpec",
    "ConfigError",
    "EngineConfig",
    "ModelSpec",
    "RMSNormSpec",
    "RotarySpec",
    "ScheduleEntry",
    "SwiGLUSpec",
    "architecture_name",
    "architectures",
    "canonical_dtype",
    "get_architecture",
    "load_model_config",
    "read_config_json",
    "register_architecture",
]
