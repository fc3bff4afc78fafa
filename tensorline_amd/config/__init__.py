from tensorline_amd.config.engine_config import EngineConfig, normalize_dtype  # noqa: F401
from tensorline_amd.config.model_config import ConfigError, Qwen2Config  # noqa: F401
from tensorline_amd.config.registry import (  # noqa: F401
    Architecture, get_architecture, known_architectures, load_model_config, register_architecture)
from tensorline_amd.config.samovik_config import SamovikConfig  # noqa: F401
from tensorline_amd.config.tumitar_config import TumitarConfig  # noqa: F401
from tensorline_amd.config.zeganex_config import ZeganexConfig  # noqa: F401
from tensorline_amd.config.kabulix_config import KabulixConfig  # noqa: F401
