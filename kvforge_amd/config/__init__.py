from kvforge_amd.config.engine import (CacheConfig, EngineConfig, SchedulerConfig,
                                       SchedulingPolicy, parse_dtype, DTYPES)
from kvforge_amd.config.model import (ConfigError, LlamaConfig, ModelConfig, RopeScaling,
                                      read_config_json)
from kvforge_amd.config.presets import PRESETS, preset_dict

__all__ = ["CacheConfig", "EngineConfig", "SchedulerConfig", "SchedulingPolicy", "parse_dtype",
           "DTYPES", "ConfigError", "LlamaConfig", "ModelConfig", "RopeScaling",
           "read_config_json", "PRESETS", "preset_dict"]
