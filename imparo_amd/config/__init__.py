from .errors import ConfigError, UnknownArchitecture, MissingKey, BadValue, Inconsistent
from .plan import PartSpec, LayerPlan, LayerCall, ModelPlan, pre_norm_layer
from .registry import (register_architecture, known_architectures, architecture_of,
                       read_config_json, plan_from_config)
from . import lfm2 as _lfm2
from .lfm2 import Lfm2Config, adjusted_ff_dim

register_architecture(_lfm2.ARCHITECTURE, Lfm2Config.from_dict, _lfm2.build_plan)
from . import tumadra as _tumadra
from .tumadra import TumadraConfig

register_architecture(_tumadra.ARCHITECTURE, TumadraConfig.from_dict, _tumadra.build_plan)
from . import pupalorn as _pupalorn
from .pupalorn import PupalornConfig

register_architecture(_pupalorn.ARCHITECTURE, PupalornConfig.from_dict, _pupalorn.build_plan)
from . import kosalorn as _kosalorn
from .kosalorn import KosalornConfig

register_architecture(_kosalorn.ARCHITECTURE, KosalornConfig.from_dict, _kosalorn.build_plan)
from . import mepapel as _mepapel
from .mepapel import MepapelConfig

register_architecture(_mepapel.ARCHITECTURE, MepapelConfig.from_dict, _mepapel.build_plan)
