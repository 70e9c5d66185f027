from kvforge_amd.config.engine import (CacheConfig, EngineConfig, SchedulerConfig,
                                       SchedulingPolicy, parse_dtype, DTYPES)
from kvforge_amd.config.model import (ConfigError, LlamaConfig, ModelConfig, RopeScaling,
                                      read_config_json)
from kvforge_amd.config.fogorax import FogoraxConfig
from kvforge_amd.config.rudorax import RudoraxConfig
from kvforge_amd.config.buzinex import BuzinexConfig
from kvforge_amd.config.ludelix import LudelixConfig
from kvforge_amd.config.presets import PRESETS, preset_dict

__all__ = ["CacheConfig", "EngineConfig", "SchedulerConfig", "SchedulingPolicy", "parse_dtype",
           "DTYPES", "ConfigError", "FogoraxConfig", "RudoraxConfig", "BuzinexConfig", "LudelixConfig", "LlamaConfig", "ModelConfig", "RopeScaling",
           "read_config_json", "PRESETS", "preset_dict"]
