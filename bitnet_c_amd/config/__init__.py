"""Typed configurations and the architecture registry; importing registers "llama", "Sunusun", "Sonodra", "Fazopel" and "Mutirax"."""
from .base import (Architecture, ConfigError, architecture_for, architecture_names, load_config,
                   read_config_json, register_architecture)
from .llama import LlamaConfig, RopeScaling
from .sunusun import SunusunConfig
from .sonodra import SonodraConfig
from .fazopel import FazopelConfig
from .mutirax import MutiraxConfig
from . import llama_plan  # noqa: F401  (registration)
