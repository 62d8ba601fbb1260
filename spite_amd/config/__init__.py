from .llama4 import Llama4Config, RopeScaling, ConfigError
from .registry import (register_architecture, architecture, registered_architectures, read_config,
                       UnknownArchitecture, Architecture)
from .ravenex import RavenexConfig
from .pefedra import PefedraConfig
from .tebalorn import TebalornConfig
from .nolapel import NolapelConfig
from . import llama4_spec  # noqa: F401  (registers Llama4ForCausalLM)
from . import ravenex_spec  # noqa: F401  (registers Ravenex)
from . import pefedra_spec  # noqa: F401  (registers Pefedra)
from . import tebalorn_spec  # noqa: F401  (registers Tebalorn)
from . import nolapel_spec  # noqa: F401  (registers Nolapel)
