from .spec import (ConfigError, LayerSpec, ModelSpec, PartSpec, ScheduleEntry,
                   default_schedule)
from .lfm2 import Lfm2Config
from .koketar import KoketarConfig
from .vavelorn import VavelornConfig
from .dalerax import DaleraxConfig
from .telapel import TelapelConfig
from .registry import (architecture_name, config_from_dict, load_config,
                       register_architecture, registered_architectures)

register_architecture("Lfm2ForCausalLM", Lfm2Config)
register_architecture("lfm2", Lfm2Config)
register_architecture("Koketar", KoketarConfig)
register_architecture("Vavelorn", VavelornConfig)
register_architecture("Dalerax", DaleraxConfig)
register_architecture("Telapel", TelapelConfig)

__all__ = [
    "ConfigError", "LayerSpec", "ModelSpec", "PartSpec", "ScheduleEntry", "default_schedule",
    "Lfm2Config", "KoketarConfig", "VavelornConfig", "DaleraxConfig", "TelapelConfig", "architecture_name", "config_from_dict", "load_config",
    "register_architecture", "registered_architectures",
]
