from tensorline_amd.config.engine_config import EngineConfig, normalize_dtype  # noqa: F401
from tensorline_amd.config.model_config import ConfigError, Qwen2Config  # noqa: F401
from tensorline_amd.config.registry import (  # noqa: F401
    Architecture, get_architecture, known_architectures, load_model_config, register_architecture)
