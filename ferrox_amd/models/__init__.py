from .registry import Architecture, config_from_folder, known_architectures, register_architecture, resolve

__all__ = ["Architecture", "config_from_folder", "known_architectures", "register_architecture", "resolve"]
