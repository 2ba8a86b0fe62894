"""cpm.cu_amd: a small generation engine (MiniCPM4, Duvulix, Gumodra) for one AMD MI355X (gfx950).

Importable as ``cpmcu_amd`` (the folder name ``cpm.cu_amd`` is not a Python
identifier; ``cpmcu_amd`` beside it is a link to the same folder).
"""
from . import models  # registers the built-in architectures and parts
from .config import ConfigError, DuvulixConfig, GumodraConfig, MiniCPMConfig
from .engine import Engine, EngineOptions, StepEntry, StepError
from .registry import architectures, get_architecture, register_architecture

__all__ = ["Engine", "EngineOptions", "StepEntry", "StepError", "ConfigError", "MiniCPMConfig", "DuvulixConfig", "GumodraConfig",
           "architectures", "get_architecture", "register_architecture"]
