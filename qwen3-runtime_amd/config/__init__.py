from .engine import EngineConfig  # noqa: F401
from .model import ConfigError, Qwen3Config, read_config_json  # noqa: F401
from .presets import PRESETS, preset  # noqa: F401
