"""The one registry from an architecture's name to its configuration class and
its model description.  Unknown names fail closed, naming the string
(ferrox-models/src/capability.rs:603-612, loader.rs:122-123)."""
from __future__ import annotations

from dataclasses import dataclass
from typing import Callable

from ..config.base import ConfigError, read_config_json


@dataclass(frozen=True)
class Architecture:
    """One entry of the registry.

    `name` is what config.json gives as `architectures[0]`, `model_type` its `model_type`.
    `config_class` is the typed configuration: it must offer the class method
    `from_dict(raw: dict, where: str = ...)`, which reads and validates the keys of config.json (raising
    `ConfigError`), and `to_dict()`, which gives them back for a config.json to be written; it may offer
    `defaulted_keys` (names of keys that were absent and got defaults), which the command line reports.
    Nothing else of it is looked at outside `build_spec`.
    `build_spec(config, tensor_names or None) -> ModelSpec` turns it into the model's description."""
    name: str
    model_type: str
    config_class: type
    build_spec: Callable


_BY_NAME: dict[str, Architecture] = {}
_BY_TYPE: dict[str, Architecture] = {}


def register_architecture(arch: Architecture) -> None:
    for method in ("from_dict", "to_dict"):
        if not callable(getattr(arch.config_class, method, None)):
            raise TypeError(f"architecture '{arch.name}': its configuration class has no {method}()")
    _BY_NAME[arch.name] = arch
    _BY_TYPE[arch.model_type] = arch


def architecture_of(config) -> Architecture:
    """The registered architecture whose configuration class `config` is an instance of."""
    for arch in _BY_NAME.values():
        if isinstance(config, arch.config_class):
            return arch
    raise ConfigError(f"no registered architecture has a configuration of type {type(config).__name__}")


def known_architectures():
    return sorted(_BY_NAME)


def resolve(raw_config: dict) -> Architecture:
    """By `architectures[0]`, else by `model_type`."""
    archs = raw_config.get("architectures")
    if isinstance(archs, list) and archs:
        if archs[0] in _BY_NAME:
            return _BY_NAME[archs[0]]
        raise ConfigError(f"unsupported architecture '{archs[0]}' (known: {', '.join(known_architectures())})")
    mt = raw_config.get("model_type")
    if mt in _BY_TYPE:
        return _BY_TYPE[mt]
    raise ConfigError(f"config.json names no known architecture (architectures={archs!r}, model_type={mt!r}; "
                      f"known: {', '.join(known_architectures())})")


def config_from_folder(folder: str):
    raw = read_config_json(folder)
    arch = resolve(raw)
    return arch, arch.config_class.from_dict(raw, where=f"{folder}/config.json")


def _register_builtin():
    from ..config.qwen2_moe import Qwen2MoeConfig
    from .qwen2_moe import build_spec
    register_architecture(Architecture(Qwen2MoeConfig.architecture, Qwen2MoeConfig.model_type,
                                       Qwen2MoeConfig, build_spec))


_register_builtin()
