"""ferrox_amd: a one-GPU inference engine for the Qwen2-MoE architecture on MI355X."""
from . import parts  # noqa: F401  (registers the built-in parts)
from .config import ConfigError, Qwen2MoeConfig
from .models import config_from_folder, known_architectures, register_architecture

__all__ = ["ConfigError", "Qwen2MoeConfig", "config_from_folder", "known_architectures", "register_architecture"]
__version__ = "0.1.0"
