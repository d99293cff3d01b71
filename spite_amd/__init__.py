"""spite_amd: a small, whole Llama 4 inference engine for one AMD MI355X (gfx950)."""
from .config import Llama4Config, ConfigError, read_config, register_architecture, registered_architectures
from .engine.engine import Engine, StepEntry, EngineError
from .sampling.sampler import SamplingParams

__all__ = ["Engine", "StepEntry", "EngineError", "SamplingParams", "Llama4Config", "ConfigError", "read_config",
           "register_architecture", "registered_architectures"]
