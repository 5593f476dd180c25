from .plan import ConfigError, LayerPlan, ModelPlan, PartSpec, ScheduleEntry
from .registry import (architecture_name, config_from_dict, load_config,
                       register_architecture, registered_architectures)
from .gemma2 import Gemma2Config
from .novotar import NovotarConfig
from .telulorn import TelulornConfig
from .pefitar import PefitarConfig
from .vifirax import VifiraxConfig
from . import presets

register_architecture("Gemma2ForCausalLM", Gemma2Config, model_type="gemma2")
register_architecture("Novotar", NovotarConfig)
register_architecture("Telulorn", TelulornConfig)
register_architecture("Pefitar", PefitarConfig)
register_architecture("Vifirax", VifiraxConfig)
