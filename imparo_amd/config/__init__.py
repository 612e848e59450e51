from .errors import ConfigError, UnknownArchitecture, MissingKey, BadValue, Inconsistent
from .plan import PartSpec, LayerPlan, LayerCall, ModelPlan, pre_norm_layer
from .registry import (register_architecture, known_architectures, architecture_of,
                       read_config_json, plan_from_config)
from . import lfm2 as _lfm2
from .lfm2 import Lfm2Config, adjusted_ff_dim

register_architecture(_lfm2.ARCHITECTURE, Lfm2Config.from_dict, _lfm2.build_plan)
