"""cpm.cu_amd: a small MiniCPM4 generation engine for one AMD MI355X (gfx950).

Importable as ``cpmcu_amd`` (the folder name ``cpm.cu_amd`` is not a Python
identifier; ``cpmcu_amd`` beside it is a link to the same folder).
"""
from . import models  # registers the built-in architectures and parts
from .config import ConfigError, MiniCPMConfig
from .engine import Engine, EngineOptions, StepEntry, StepError
from .registry import architectures, get_architecture, register_architecture

__all__ = ["Engine", "EngineOptions", "StepEntry", "StepError", "ConfigError", "MiniCPMConfig",
           "architectures", "get_architecture", "register_architecture"]
