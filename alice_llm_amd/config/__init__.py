from .plan import ConfigError, LayerPlan, ModelPlan, PartSpec, ScheduleEntry
from .registry import (architecture_name, config_from_dict, load_config,
                       register_architecture, registered_architectures)
from .gemma2 import Gemma2Config
from . import presets

register_architecture("Gemma2ForCausalLM", Gemma2Config, model_type="gemma2")
