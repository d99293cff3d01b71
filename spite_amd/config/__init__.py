from .llama4 import Llama4Config, RopeScaling, ConfigError
from .registry import (register_architecture, architecture, registered_architectures, read_config,
                       UnknownArchitecture, Architecture)
from . import llama4_spec  # noqa: F401  (registers Llama4ForCausalLM)
