"""Typed configurations and the registry of architectures.  An architecture's own configuration class lives in
its own module (`cwm_amd.config.llama3` for the Llama-3 dense decoder) and is not exported from here."""

from .schema import ConfigError, from_dict, to_dict
from .registry import (
    ARCHITECTURES,
    Architecture,
    get_architecture,
    load_config,
    parse_config,
    register_architecture,
)

__all__ = [
    "ConfigError",
    "from_dict",
    "to_dict",
    "ARCHITECTURES",
    "Architecture",
    "get_architecture",
    "load_config",
    "parse_config",
    "register_architecture",
]
