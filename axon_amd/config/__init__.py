from .base import (ConfigError, LayerSpec, ModelConfig, ModelSpec, PartSpec, Run, read_config_json)
from .engine import EngineConfig, dtype_name
from .registry import (architecture_of, config_from_dict, config_from_dir, known_architectures,
                       register_architecture)
from .qwen2 import Qwen2Config
from .pikesun import PikesunConfig
from .figalorn import FigalornConfig
from .napizen import NapizenConfig
from .zugutar import ZugutarConfig

__all__ = ["ConfigError", "LayerSpec", "ModelConfig", "ModelSpec", "PartSpec", "Run", "read_config_json",
           "EngineConfig", "dtype_name", "architecture_of", "config_from_dict", "config_from_dir",
           "known_architectures", "register_architecture", "Qwen2Config", "PikesunConfig", "FigalornConfig", "NapizenConfig", "ZugutarConfig"]

register_architecture(Qwen2Config.architecture, Qwen2Config, Qwen2Config.model_type)
register_architecture(PikesunConfig.architecture, PikesunConfig, PikesunConfig.model_type)
register_architecture(FigalornConfig.architecture, FigalornConfig, FigalornConfig.model_type)
register_architecture(NapizenConfig.architecture, NapizenConfig, NapizenConfig.model_type)
register_architecture(ZugutarConfig.architecture, ZugutarConfig, ZugutarConfig.model_type)
