from .llama import ConfigError, LlamaConfig, RopeScaling
from .registry import (config_from_dict, config_from_folder, register_architecture, registered_architectures,
                       unregister_architecture)
from .bovozen import BovozenConfig
from .gedunex import GedunexConfig
from .rekirax import RekiraxConfig
from .situlorn import SitulornConfig
from .spec import LayerSpec, ModelSpec, PartSpec, ScheduleEntry

__all__ = ["BovozenConfig", "ConfigError", "GedunexConfig", "LlamaConfig", "RekiraxConfig", "RopeScaling", "SitulornConfig", "config_from_dict", "config_from_folder",
           "register_architecture", "registered_architectures", "unregister_architecture", "LayerSpec", "ModelSpec",
           "PartSpec", "ScheduleEntry"]
