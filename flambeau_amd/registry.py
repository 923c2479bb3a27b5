"""One registry from the architecture's name (``config.json``'s ``architectures[0]``) to
its typed configuration and its model description.

The reference's registry maps an architecture string to a handler and names the known ones
when asked for an unknown one (crates/runtime/src/registry.rs:18-77)."""
from __future__ import annotations

from dataclasses import dataclass
from typing import Callable

from .config.base import ConfigError, architecture_name, read_config_json


class UnknownArchitecture(ConfigError):
    pass


@dataclass
class Architecture:
    name: str
    config_class: type                # has from_dict(raw, where)
    build_spec: Callable              # config -> models.decoder.ModelSpec


_ARCHITECTURES: dict[str, Architecture] = {}


def register_architecture(name: str, config_class, build_spec) -> None:
    _ARCHITECTURES[name] = Architecture(name, config_class, build_spec)


def known_architectures() -> list[str]:
    _load_builtin()
    return sorted(_ARCHITECTURES)


def find_architecture(name: str) -> Architecture:
    _load_builtin()
    try:
        return _ARCHITECTURES[name]
    except KeyError:
        raise UnknownArchitecture(
            f"unknown architecture '{name}'; known: {', '.join(sorted(_ARCHITECTURES)) or '(none)'}") from None


def config_from_dict(raw: dict, where: str = "config.json"):
    """``(Architecture, typed config)`` for a config.json dictionary."""
    arch = find_architecture(architecture_name(raw, where))
    return arch, arch.config_class.from_dict(raw, where)


def config_from_dir(model_dir):
    raw = read_config_json(model_dir)
    return config_from_dict(raw, f"{model_dir}/config.json")


def _load_builtin():
    from . import models
    models.discover()           # every module under models/ registers its architecture
