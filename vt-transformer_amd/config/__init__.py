from .base import ConfigError, LayerSpec, ModelConfig, ModelSpec, PartSpec, ScheduleEntry
from .registry import architectures, config_from_dict, load_config, register_architecture
from .qwen2 import Qwen2Config
from .lisunex import LisunexConfig
from .gabelorn import GabelornConfig
from .kigalix import KigalixConfig
from .fedovik import FedovikConfig

register_architecture(Qwen2Config.architecture, Qwen2Config)
register_architecture(LisunexConfig.architecture, LisunexConfig)
register_architecture(GabelornConfig.architecture, GabelornConfig)
register_architecture(KigalixConfig.architecture, KigalixConfig)
register_architecture(FedovikConfig.architecture, FedovikConfig)

__all__ = ["ConfigError", "LayerSpec", "ModelConfig", "ModelSpec", "PartSpec", "ScheduleEntry",
           "architectures", "config_from_dict", "load_config", "register_architecture", "Qwen2Config", "LisunexConfig", "GabelornConfig",
           "KigalixConfig", "FedovikConfig"]
