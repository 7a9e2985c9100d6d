"""Typed configuration and the architecture registry."""
from .registry import (ConfigError, config_from_dict, config_from_dir, read_config_json,
                       register_architecture, registered_architectures, resolve_architecture)
from .spec import ExecEntry, LayerSpec, ModelSpec, PartSpec, default_schedule
from .minicpm import MiniCPMConfig, RopeScaling

__all__ = [
    "ConfigError", "config_from_dict", "config_from_dir", "read_config_json",
    "register_architecture", "registered_architectures", "resolve_architecture",
    "ExecEntry", "LayerSpec", "ModelSpec", "PartSpec", "default_schedule",
    "MiniCPMConfig", "RopeScaling",
]
