from tokasaurus_amd.config.engine_config import EngineConfig, OptionError, apply_overrides  # noqa: F401
from tokasaurus_amd.config.model_config import ConfigError, LlamaConfig, RopeScaling  # noqa: F401
