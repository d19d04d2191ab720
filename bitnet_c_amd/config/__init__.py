"""Typed configurations and the architecture registry; importing registers "llama"."""
from .base import (Architecture, ConfigError, architecture_for, architecture_names, load_config,
                   read_config_json, register_architecture)
from .llama import LlamaConfig, RopeScaling
from . import llama_plan  # noqa: F401  (registration)
